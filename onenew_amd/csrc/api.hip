// Kernel-level C ABI (include/onenew_hip.h): argument checks, geometry set-up and kernel choice.
// Device pointers in, asynchronous launches on the caller's stream, no allocation except the
// lazily grown split-K scratch.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <math.h>
#include <stdlib.h>

#include <atomic>
#include <map>
#include <mutex>
#include <vector>

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
    e.qlut = nullptr;
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
static long long g_scratch_generation = 0;   // how many blocks have been allocated so far

// ---- the entry point that allocates nothing ------------------------------------------------------
// Its split-K partial sums go to a device array that is part of the code object: every GPU the library runs on holds
// its own copy for the life of the process.  The name `scratch` is a host-side handle, not a device address: host code
// asks the runtime for the array's address once per device and passes that on.
static const size_t kNoAllocScratchBytes = (size_t) 32 << 20;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
static const int kMaxDevices = 64;
static void *g_noalloc_ptr[kMaxDevices];      // address of `scratch` on each device, once looked up there
static thread_local void *tl_noalloc = nullptr;   // non-null while this thread runs the entry point: get_scratch hands it out
static std::atomic<long long> g_noalloc_scratch_uses{0};   // launches whose partial sums went to the built-in array

// address of this device's copy of `scratch`; looked up with that device current, no allocation involved
static int noalloc_scratch(void **out) {
    int dev = -1;
    ONHIP_CHECK_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return set_error(ONHIP_ERR_RUNTIME, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_noalloc_ptr[dev]) {
        void *ptr = nullptr;
        ONHIP_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return set_error(ONHIP_ERR_RUNTIME, "no device address for the built-in scratch array");
        g_noalloc_ptr[dev] = ptr;
    }
    *out = g_noalloc_ptr[dev];
    return ONHIP_OK;
}

static int get_scratch(size_t bytes, void **out) {
    if (tl_noalloc) {
        if (bytes > kNoAllocScratchBytes)
            return set_error(ONHIP_ERR_WORKSPACE, "conv (no allocation): the split-K partial sums of this problem take %zu bytes, "
                             "the built-in scratch holds %zu; use onhip_conv2d_f32", bytes, kNoAllocScratchBytes);
        *out = tl_noalloc;
        g_noalloc_scratch_uses.fetch_add(1, std::memory_order_relaxed);
        return ONHIP_OK;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (bytes > g_scratch_bytes) {
        // A HIP graph recorded by a caller holds the current block's address in its kernel arguments, and its replays
        // keep writing and reading partial sums there: a block that is outgrown is kept until the process ends (the
        // replays then have it to themselves), never freed.  Sizes at least double, so all retired blocks together are
        // smaller than the live one.
        size_t want = bytes < (64u << 20) ? (64u << 20) : bytes;
        if (want < 2 * g_scratch_bytes) want = 2 * g_scratch_bytes;
        void *fresh = nullptr;
        ONHIP_CHECK_HIP(hipMalloc(&fresh, want));
        g_scratch = fresh;
        g_scratch_bytes = want;
        ++g_scratch_generation;
    }
    *out = g_scratch;
    return ONHIP_OK;
}

// Workspace of the split-K reduction that runs inside the launch: partial sums and one arrival counter per tile in
// uncached device memory, so that what one XCD wrote is what another reads without flushing anybody's L2.  Allocated
// once at first use and kept for the life of the process.
static void *g_uc = nullptr;
static int *g_arrive = nullptr;
static const size_t kUcBytes = (size_t) 256 << 20;
static bool g_arrive_dirty = false;   // a launch that counts arrivals failed: the counters may not be back at zero
static int get_uc(void **buf, int **arrive) {
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_arrive && g_arrive_dirty) {
        ONHIP_CHECK_HIP(hipDeviceSynchronize());
        ONHIP_CHECK_HIP(hipMemset(g_arrive, 0, 4 << 20));
        ONHIP_CHECK_HIP(hipDeviceSynchronize());
        g_arrive_dirty = false;
    }
    if (!g_uc || !g_arrive) {   // both or neither: a call that fails half-way leaves what it got for the next one
        if (!g_uc) ONHIP_CHECK_HIP(hipExtMallocWithFlags(&g_uc, kUcBytes, hipDeviceMallocUncached));
        void *ctr = nullptr;
        ONHIP_CHECK_HIP(hipExtMallocWithFlags(&ctr, 4 << 20, hipDeviceMallocUncached));
        ONHIP_CHECK_HIP(hipMemset(ctr, 0, 4 << 20));
        ONHIP_CHECK_HIP(hipDeviceSynchronize());
        g_arrive = static_cast<int *>(ctr);
    }
    *buf = g_uc; *arrive = g_arrive;
    return ONHIP_OK;
}

// ---- tile and split-K choice ----------------------------------------------------------------------
//
// A launch is described by (tile BM x BN, split): split > 1 cuts K into slices that write partial
// sums to the scratch buffer and a finishing kernel adds them up.  The choice comes from a cost model
// or, when tuning is on, from timing the candidates once per problem signature (the counterpart of
// the reference's grid search over GEMM tiles, tools/optimize/auto_tuning.hpp:9-75).
static const int kTiles[][2] = {{128, 128}, {64, 128}, {64, 64}, {32, 128}};
static const int kNumTiles = 4;
static const int kSplits[] = {1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 16, 24, 32};
static const int kNumSplits = 13;

// tail > 1: the tiles left over after whole rounds of 256 are cut `tail` ways along K (launch_choice)
// rowb != 0: the kernel that feeds B from global memory straight into the MFMAs (igemm_rowb.hip), tile bm x bn
// fin != 0 (with split > 1 or tail > 1): the slices of a tile are added up by the last of them to arrive, inside the
// launch, instead of by a finishing launch (igemm_kernel, `arrive`)
// dma != 0: the kernel that loads its operand tiles straight into LDS (igemm_dma_kernel.hpp), tile bm x bn, never split;
// 1 = ring of stages within 64 KiB of LDS, 2 = the long ring
struct Choice { int bm, bn, split, tail, rowb, fin, dma; };

static std::mutex g_tune_mu;
static int g_tune_mode = -1;   // -1: read ONHIP_TUNE on first use; 0 model only; 1 measure
static std::map<std::vector<long long>, Choice> g_tuned;

static int tune_mode() {
    if (g_tune_mode < 0) {
        const char *e = getenv("ONHIP_TUNE");
        g_tune_mode = (e && atoi(e) > 0) ? 1 : 0;
    }
    return g_tune_mode;
}

// Optional persistence of measured choices: ONHIP_TUNE_CACHE names a text file, one line per problem
// signature ("v0 v1 ... v13 : bm bn split"), read once and appended to after every measurement.
static bool g_cache_loaded = false;
static void load_tune_cache_locked() {
    if (g_cache_loaded) return;
    g_cache_loaded = true;
    const char *path = getenv("ONHIP_TUNE_CACHE");
    if (!path) return;
    FILE *f = fopen(path, "r");
    if (!f) return;
    char line[512];
    while (fgets(line, sizeof(line), f)) {
        std::vector<long long> key;
        char *s = line, *end = nullptr;
        for (;;) {
            while (*s == ' ') ++s;
            if (*s == ':' || *s == 0 || *s == '\n') break;
            const long long v = strtoll(s, &end, 10);
            if (end == s) break;
            key.push_back(v);
            s = end;
        }
        Choice c = {0, 0, 1, 0, 0, 0, 0};
        if (*s == ':' && key.size() == 14 && sscanf(s + 1, "%d %d %d %d %d %d %d", &c.bm, &c.bn, &c.split, &c.tail, &c.rowb, &c.fin, &c.dma) >= 3 &&
            c.bm > 0 && c.bn > 0 && c.split >= 1 && c.split <= 64 && c.tail >= 0 && c.tail <= 64)
            g_tuned[key] = c;
    }
    fclose(f);
}
static void append_tune_cache_locked(const std::vector<long long> &key, const Choice &c) {
    const char *path = getenv("ONHIP_TUNE_CACHE");
    if (!path) return;
    FILE *f = fopen(path, "a");
    if (!f) return;
    for (long long v : key) fprintf(f, "%lld ", v);
    fprintf(f, ": %d %d %d %d %d %d %d\n", c.bm, c.bn, c.split, c.tail, c.rowb, c.fin, c.dma);
    fclose(f);
}

// 16-byte units per K tile of the deepest kernel of a data type (slices of K are whole tiles)
static int k_tile_units(int dt) { (void) dt; return 4; }

static int mfma_k_per_unit(int dt) { return dt == DT_F32 ? 4 : dt == DT_I8 ? 16 : 8; }

// cycles one CU needs for the MFMAs of one K tile of a BM x BN workgroup
static double tile_mfma_cycles(int dt, int bm, int bn) {
    const double flops = 2.0 * bm * bn * 4 * mfma_k_per_unit(dt);
    const double per_clk = dt == DT_F32 ? 256.0 : dt == DT_I8 ? 8192.0 : 4096.0;
    return flops / per_clk;
}

static int apply_choice(IgemmLaunch &cfg, IgemmParams &p, const Choice &c) {
    cfg.bm = c.bm; cfg.bn = c.bn; cfg.split = 1;
    p.k_split_units = p.k_units;
    p.partial = nullptr;
    if (c.split > 1) {
        const int upt = k_tile_units(cfg.dtype);
        const int k_tiles = (p.k_units + upt - 1) / upt;
        const int tiles_per = (k_tiles + c.split - 1) / c.split;
        const int split = (k_tiles + tiles_per - 1) / tiles_per;
        if (split > 1) {
            const size_t bytes = (size_t) split * cfg.batch * p.M * (p.N - p.part_begin) * 4;
            int rc;
            cfg.split = split;
            p.k_split_units = tiles_per * upt;
            p.arrive = nullptr;
            if (c.fin && cfg.dtype != DT_I8 && bytes <= kUcBytes && !tl_noalloc) {
                void *uc; int *arr;
                rc = get_uc(&uc, &arr);
                if (rc) return rc;
                p.partial = reinterpret_cast<float *>(uc);
                p.arrive = arr;
                p.n_slices = split;
            } else {
                void *buf = nullptr;
                rc = get_scratch(bytes, &buf);
                if (rc) return rc;
                p.partial = reinterpret_cast<float *>(buf);
            }
        }
    }
    return ONHIP_OK;
}

// Tile quantisation.  All workgroups of these launches are resident at once, so the CUs that hold one workgroup more
// than the others set the duration: 784 tiles on 256 CUs take as long as 1024.  When few tiles are left over after
// whole rounds of 256, the launch treats its tiles in two ways: the first dp_cols column blocks (a whole number of
// rounds) are whole tiles, each of the remaining tiles is cut along K into slices so that the leftover, too, puts about
// one small workgroup on every CU.  (Running the leftover as a second launch on another stream was tried first: the
// cross-queue event waits cost more than the balance gained.)
static bool tail_geometry(const IgemmLaunch &cfg, const IgemmParams &p, int bm, int bn, int *dp_cols, int *tail_tiles) {
    if (cfg.batch != 1 || cfg.dtype == DT_I8) return false;
    const int tiles_m = (p.M + bm - 1) / bm, cols = (p.N + bn - 1) / bn;
    const long long tiles = (long long) tiles_m * cols;
    const int rounds = (int) (tiles / 256);
    if (rounds < 1) return false;
    const int dpc = rounds * 256 / tiles_m;
    if (dpc < 1 || dpc >= cols) return false;
    const int left = (cols - dpc) * tiles_m;
    if (left > 128) return false;   // more than half a round left over: nothing to gain
    *dp_cols = dpc;
    *tail_tiles = left;
    return true;
}

static const int kRowbTiles[][2] = {{64, 128}, {128, 128}, {64, 256}, {96, 128}, {32, 256}, {32, 512}};
static const int kNumRowbTiles = 6;

// (bm, bn) is a tile this build has a kernel for
static bool tile_exists(const Choice &c) {
    if (c.dma) return c.dma <= 2 && dma_tile_ok(c.bm, c.bn);
    const int (*list)[2] = c.rowb ? kRowbTiles : kTiles;
    const int n = c.rowb ? kNumRowbTiles : kNumTiles;
    for (int t = 0; t < n; ++t)
        if (list[t][0] == c.bm && list[t][1] == c.bn) return true;
    return false;
}

static bool candidate_ok(const IgemmLaunch &cfg, const IgemmParams &p, const Choice &c) {
    if (!tile_exists(c)) return false;   // e.g. a line of the cache file written by another build or by hand
    const int k_tiles = (p.k_units + k_tile_units(cfg.dtype) - 1) / k_tile_units(cfg.dtype);
    const bool h16 = cfg.dtype != DT_I8 && (cfg.bl == BL_KVEC || cfg.bl == BL_KVEC_TAP);   // 16-bit storage: that kernel only
    // int8 with a residual operand: the register-staged kernel, whole K in one workgroup
    if (p.res && cfg.dtype == DT_I8 && (c.dma || c.split > 1 || c.tail > 1 || c.fin || c.rowb)) return false;
    if (c.dma) {
        static const bool off = getenv("ONHIP_NO_DMA") != nullptr;   // tuning hook: the register-staged kernel only
        return (!off || h16) && c.split == 1 && c.tail <= 1 && !c.rowb && !c.fin && dma_ok(cfg, p);
    }
    if (h16) return false;
    if (c.rowb && (c.split != 1 || !rowb_f32_ok(cfg, p))) return false;
    if (c.fin) {
        static const bool off = getenv("ONHIP_NO_FIN") != nullptr;   // tuning hook: finishing launches only
        if (off) return false;
        const long long tiles = (long long) ((p.M + c.bm - 1) / c.bm) * ((p.N + c.bn - 1) / c.bn) * cfg.batch;
        if (cfg.dtype == DT_I8 || c.rowb || (c.split <= 1 && c.tail <= 1) || tiles > (1 << 20)) return false;
    }
    if (c.tail > 1) {
        int dpc, left;
        return c.split == 1 && k_tiles >= 2 * c.tail && tail_geometry(cfg, p, c.bm, c.bn, &dpc, &left);
    }
    if (c.split > 1 && (k_tiles < 2 * c.split)) return false;
    if (c.split > 1 && (size_t) c.split * cfg.batch * p.M * p.N * 4 > ((size_t) 256 << 20)) return false;
    return true;
}

// Cost model (cycles).  A CU works through its share of the workgroups; co-resident workgroups share
// the MFMA pipes, so the MFMA time adds up while the per-workgroup fill/drain latency overlaps when
// several are resident.  Split-K adds the partial-sum traffic and a second launch.
static double model_cost(const IgemmLaunch &cfg, const IgemmParams &p, const Choice &c) {
    const long long tiles = (long long) ((p.M + c.bm - 1) / c.bm) * ((p.N + c.bn - 1) / c.bn) * cfg.batch;
    const int k_tiles = (p.k_units + 3) / 4;
    const int per = (k_tiles + c.split - 1) / c.split;
    const double wgs = (double) tiles * c.split;
    const double per_cu = ceil(wgs / 256.0);
    const int regs_occ = c.bm * c.bn >= 128 * 128 ? 3 : c.bm * c.bn >= 64 * 128 ? 4 : 6;
    const double resident = per_cu < regs_occ ? per_cu : regs_occ;
    // measured steady-state inefficiency; a workgroup alone on its CU (one wavefront per SIMD, in lock step at every
    // barrier) needs 690 cycles for the 512 of a K tile where several resident ones need about 600
    const double overhead = (cfg.bl == BL_GATHER ? 1.35 : 1.18) * (resident <= 1.0 ? 1.15 : 1.0);
    // fp32: the wider tiles leave fewer wavefronts resident and measure behind the 64 x 64 one wherever the two come
    // out even here (ViT-Tiny's first MLP product at batch 64: 50 against 44 us)
    const double wide = cfg.dtype == DT_F32 && c.bm * c.bn > 64 * 64 ? 1.05 : 1.0;
    const double mfma = per * tile_mfma_cycles(cfg.dtype, c.bm, c.bn) * overhead * wide;
    const double fixed = 2600.0 + 12.0 * (c.bm * c.bn / 256);     // first loads in flight + epilogue stores
    // the fixed part of co-resident workgroups overlaps; a last, partly filled group of them pays its share of it, not
    // all of it (with all of it the 64 x 128 tile won over 64 x 64 on short-K layers, where it measures 15 % slower)
    double cycles = per_cu * mfma + per_cu / resident * fixed;
    if (c.split > 1) cycles += 9000.0 + (double) (c.split + 1) * p.M * p.N * cfg.batch * 4.0 / 1500.0;
    return cycles;
}

// A tile the caller asks for (onhip_set_tile_hint): the model-wide GEMM tile a .one file carries in
// BLOCK_INFO_S.cuda_gemm_tile_{m,n} (common/nn_common.h:28-39).  While it is set on a thread, the cost model chooses
// among the splits of that tile only; measured choices (tuning mode 1) and ONHIP_TILE take precedence.
static thread_local int tl_hint_bm = 0, tl_hint_bn = 0;

// The direct-to-LDS int8 kernel where the problem allows it (measured on YOLOv8s layer shapes: about twice as fast as the
// register-staged kernel wherever it has work for most of the CUs): the largest tile that still gives every CU a
// workgroup and then some.  Problems with so few tiles that only a split along K reaches all CUs stay with the
// register-staged kernel, which has one.
static bool dma_model_choice(const IgemmLaunch &cfg, const IgemmParams &p, Choice *out) {
    static const int order[4][2] = {{128, 128}, {128, 64}, {64, 128}, {64, 64}};
    // what a tile's steady state costs per output against the largest one's (measured on the YOLOv8s layers)
    static const double eff[4] = {1.0, 1.08, 1.10, 1.20};
    const bool only = cfg.dtype != DT_I8;   // the 16-bit types have no other kernel for these operands
    // int8 with a large fp32 result (the reference's W8A32 form on big planes): the register-staged kernel's store of
    // fp32 rows is the faster one from about 6.5 million outputs up (every such YOLOv8s layer at batch 16, 5-35 %)
    if (!only && !p.out_s8 && (long long) p.M * p.N >= (long long) 256 * 25600) return false;
    // The largest tile does not always win: among the tiles that give every CU a workgroup and then some, the one with the
    // least work in its rounds of 256 workgroups (800 tiles of 128 x 128 are four rounds, 1600 of 128 x 64 seven half as
    // long).  Problems with so few tiles that only a split along K reaches all CUs go to the register-staged kernel.
    int best = -1;
    double best_cost = 1e300;
    for (int t = 0; t < 4; ++t) {
        const Choice c = {order[t][0], order[t][1], 1, 0, 0, 0, 1};
        if (!candidate_ok(cfg, p, c)) return false;
        if (c.bm == 128 && p.M <= 64) continue;
        const long long tiles = (long long) ((p.M + c.bm - 1) / c.bm) * ((p.N + c.bn - 1) / c.bn);
        if (tiles < 320 && t != 3) continue;
        if (t == 3 && tiles < 96 && p.k_units >= 128 && !only) return false;
        const double cost = (double) ((tiles + 255) / 256) * c.bm * c.bn * eff[t];
        if (cost < best_cost) { best_cost = cost; best = t; }
    }
    if (best < 0) return false;
    *out = Choice{order[best][0], order[best][1], 1, 0, 0, 0, 1};
    return true;
}

static Choice model_choice(const IgemmLaunch &cfg, const IgemmParams &p) {
    Choice best = {64, 64, 1, 0, 0, 0};
    const bool vec = cfg.bl == BL_KVEC || cfg.bl == BL_KVEC_TAP;
    if (vec && (cfg.dtype != DT_I8 || !tl_hint_bm) && dma_model_choice(cfg, p, &best)) return best;
    // int8 with a large fp32 result (see dma_model_choice): 64 x 64 on the register-staged kernel (measured 1-5 % ahead of
    // 64 x 128 on every such layer of YOLOv8s at batch 16), 32 x 128 where there are no more than 32 rows
    if (vec && cfg.dtype == DT_I8 && !tl_hint_bm && !p.out_s8 && (long long) p.M * p.N >= (long long) 256 * 25600) {
        const Choice c = {p.M <= 32 ? 32 : 64, p.M <= 32 ? 128 : 64, 1, 0, 0, 0, 0};
        if (candidate_ok(cfg, p, c)) return c;
    }
    // fp32 1x1 convolutions with at most 32 input channels (MobileNetV2's first expansions and projection): B straight from
    // memory, no LDS round trip for an operand that is used once per 32 rows (measured 10-35 % ahead of the tiled kernel on
    // every such layer at batch 64); the tile by the row count
    if (cfg.dtype == DT_F32 && cfg.bl == BL_PLAIN && p.K <= 32 && !tl_hint_bm && !p.res) {
        const Choice c = p.M <= 32 ? Choice{32, 256, 1, 0, 1, 0, 0} : p.M % 96 == 0 ? Choice{96, 128, 1, 0, 1, 0, 0} : Choice{64, 256, 1, 0, 1, 0, 0};
        const long long tiles = (long long) ((p.M + c.bm - 1) / c.bm) * ((p.N + c.bn - 1) / c.bn);
        if (tiles >= 512 && candidate_ok(cfg, p, c)) return c;   // measured at batch 64 only: at least two workgroups per CU
    }
    for (int pass = tl_hint_bm ? 0 : 1; pass < 2; ++pass) {   // pass 0: the hinted tile; pass 1: every tile
        double best_cost = 1e300;
        for (int t = 0; t < kNumTiles; ++t)
            for (int s = 0; s < kNumSplits; ++s) {
                const Choice c = {kTiles[t][0], kTiles[t][1], kSplits[s], 0, 0, 0};
                if (pass == 0 && (c.bm != tl_hint_bm || c.bn != tl_hint_bn)) continue;
                if (!candidate_ok(cfg, p, c)) continue;
                const double cost = model_cost(cfg, p, c);
                if (cost < best_cost) { best_cost = cost; best = c; }
            }
        if (best_cost < 1e300) break;
    }
    // What measuring the candidates keeps finding on top of the tile and split above (fp32, one batch slice):
    //  * no split, and a few tiles left over after whole rounds of 256: those tiles alone cut along K so that the leftover,
    //    too, puts about a workgroup on every compute unit (launch_choice);
    //  * K slices added up by the last slice of a tile to arrive instead of by a finishing launch, where the launch has
    //    tiles enough that those last arrivers spread over the chip (at batch 1, with a handful of tiles, the finishing
    //    launch's spread over every compute unit wins).  Same sums in the same order either way.
    if (cfg.dtype == DT_F32 && !vec && !best.rowb && !best.dma) {
        int dpc = 0, left = 0;
        // ... where K is long enough to be cut: measured on the ResNet-50 layers at batch 32, a leftover cut along a K of
        // 256 or less loses 2-7 us on every layer (the slices are all fill and drain), one of 512 gains only when cut in
        // at most four
        if (best.split == 1 && p.k_units > 64 && tail_geometry(cfg, p, best.bm, best.bn, &dpc, &left)) {
            int want = 256 / left;
            want = want > 16 ? 16 : want;
            if (p.k_units <= 128 && want > 4) want = 4;
            for (int ts = want; ts >= 2; ts /= 2) {
                const Choice c = {best.bm, best.bn, 1, ts, 0, 0, 0};
                if (candidate_ok(cfg, p, c)) { best = c; break; }
            }
        }
        const long long tiles = (long long) ((p.M + best.bm - 1) / best.bm) * ((p.N + best.bn - 1) / best.bn);
        if ((best.split > 1 || best.tail > 1) && tiles >= 128) {
            Choice c = best;
            c.fin = 1;
            if (candidate_ok(cfg, p, c)) best = c;
        }
    }
    return best;
}

static std::atomic<long long> g_tail_launches{0};
static std::atomic<long long> g_dma_launches{0};

// what the calling thread's last implicit-GEMM launch ran as (onhip_last_launch_choice): tile, K slices as launched,
// slices of the leftover tiles, and which kernel
static thread_local int tl_last_choice[7] = {0, 0, 0, 0, 0, 0, 0};

// Runs the problem the way the choice says.
static int launch_choice(IgemmLaunch cfg, IgemmParams p, const Choice &c, hipStream_t st) {
    int dpc = 0, left = 0;
    p.part_begin = p.dp_tiles = p.tail_tiles = 0;
    struct Note {   // filled in on every way out of this function
        const IgemmLaunch &cfg; const IgemmParams &p; const Choice &c;
        ~Note() {
            const bool tail = p.tail_tiles > 0;
            const int v[7] = {c.bm, c.bn, c.dma || tail ? 1 : cfg.split, tail ? cfg.split : 0, c.dma ? 0 : c.rowb, p.arrive ? 1 : 0, c.dma};
            for (int i = 0; i < 7; ++i) tl_last_choice[i] = v[i];
        }
    } note{cfg, p, c};
    if (c.dma) {
        cfg.bm = c.bm; cfg.bn = c.bn; cfg.split = 1;
        cfg.ring = c.dma > 1;
        p.k_split_units = p.k_units;
        p.partial = nullptr;
        p.arrive = nullptr;
        g_dma_launches.fetch_add(1, std::memory_order_relaxed);
        return dma_launch(cfg, p, st);
    }
    auto launch = [&]() {
        const int rc = c.rowb ? rowb_f32_launch(cfg, p, st) : igemm_launch(cfg, p, st);
        if (rc && p.arrive) {   // whatever part of the launch ran may have left arrival counters above zero
            std::lock_guard<std::mutex> lock(g_scratch_mu);
            g_arrive_dirty = true;
        }
        return rc;
    };
    if (c.tail <= 1 || !tail_geometry(cfg, p, c.bm, c.bn, &dpc, &left)) {
        const Choice plain = {c.bm, c.bn, c.rowb ? 1 : c.split, 0, 0, c.rowb ? 0 : c.fin};
        int rc = apply_choice(cfg, p, plain);
        return rc ? rc : launch();
    }
    // one launch: dpc column blocks as whole tiles, the rest in c.tail K slices each; partial sums and the
    // finishing pass cover the columns from dpc * bn on only
    p.part_begin = dpc * c.bn;
    const Choice tail = {c.bm, c.bn, c.tail, 0, 0, c.rowb ? 0 : c.fin};
    int rc = apply_choice(cfg, p, tail);
    if (rc) return rc;
    if (cfg.split <= 1) {
        p.part_begin = 0;
        return launch();
    }
    p.dp_tiles = dpc * ((p.M + c.bm - 1) / c.bm);
    p.tail_tiles = left;
    g_tail_launches.fetch_add(1, std::memory_order_relaxed);
    return launch();
}

static int time_choice(IgemmLaunch cfg, IgemmParams p, const Choice &c, hipStream_t st, hipEvent_t e0, hipEvent_t e1,
                       float *best_ms) {
    int rc = launch_choice(cfg, p, c, st);   // warm-up
    if (rc) return rc;
    float best = 1e30f;
    for (int rep = 0; rep < 2; ++rep) {
        ONHIP_CHECK_HIP(hipEventRecord(e0, st));
        for (int i = 0; i < 3; ++i) {
            rc = launch_choice(cfg, p, c, st);
            if (rc) return rc;
        }
        ONHIP_CHECK_HIP(hipEventRecord(e1, st));
        ONHIP_CHECK_HIP(hipEventSynchronize(e1));
        float ms = 0.f;
        ONHIP_CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
        if (ms < best) best = ms;
    }
    *best_ms = best / 3.0f;
    return ONHIP_OK;
}

// Chooses tile, split and tail handling for the problem and launches it.
static int plan_and_launch(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t st) {
    // the entry point that allocates nothing: the cost model's choice (never the in-launch reduction, whose uncached
    // workspace is allocated on first use; no measuring, which creates events and may grow buffers)
    if (tl_noalloc) return launch_choice(cfg, p, model_choice(cfg, p), st);
    if (const char *env = getenv("ONHIP_TILE")) {   // tuning hook: ONHIP_TILE=BMxBN[xSPLIT[xTAIL[xROWB[xFIN[xDMA]]]]]
        Choice c = {0, 0, 1, 0, 0, 0, 0};
        if (sscanf(env, "%dx%dx%dx%dx%dx%dx%d", &c.bm, &c.bn, &c.split, &c.tail, &c.rowb, &c.fin, &c.dma) >= 2) {
            if (cfg.dtype != DT_I8 && (cfg.bl == BL_KVEC || cfg.bl == BL_KVEC_TAP)) {   // 16-bit storage: one kernel, its tiles
                c = {c.bm, c.bn, 1, 0, 0, 0, c.dma > 1 ? 2 : 1};
                if (!candidate_ok(cfg, p, c)) c = model_choice(cfg, p);
            }
            if (c.dma && !candidate_ok(cfg, p, c)) {   // not a problem (or a tile) for that kernel: the register-staged one
                c.dma = 0;
                if (c.bm == 128 && c.bn == 64) c.bm = 64;
            }
            if (c.fin && !candidate_ok(cfg, p, c)) c.fin = 0;
            if (c.rowb && !candidate_ok(cfg, p, c)) {   // not a problem for that kernel: the tiled one, same tile if it has it
                c.rowb = 0;
                if (c.bn > 128) c.bn = 128;
                if (c.bm == 96) c.bm = 64;
            }
            if (c.tail > 1 && !candidate_ok(cfg, p, c)) c.tail = 0;   // no leftover to split on this shape
            return launch_choice(cfg, p, c, st);
        }
    }
    if (!tune_mode()) return launch_choice(cfg, p, model_choice(cfg, p), st);
    std::vector<long long> key = {cfg.dtype, cfg.bl, cfg.batch, p.M, p.N, p.K, p.k_units, p.khkw, p.sh, p.sw,
                                  p.H, p.W, p.out_mode + (p.res ? 16 : 0), p.lda};   // a residual operand narrows the kernels
    {
        std::unique_lock<std::mutex> lock(g_tune_mu);
        load_tune_cache_locked();
        auto it = g_tuned.find(key);
        if (it != g_tuned.end()) {
            const Choice c = it->second;
            if (candidate_ok(cfg, p, c)) {
                lock.unlock();
                return launch_choice(cfg, p, c, st);
            }
            g_tuned.erase(it);   // a line of the cache file that this build would not have written: measure again
        }
    }
    // measure: the candidates the model ranks within 2.5x of its best, on the caller's stream
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone)
        return launch_choice(cfg, p, model_choice(cfg, p), st);
    const Choice guess = model_choice(cfg, p);
    const double guess_cost = model_cost(cfg, p, guess);
    hipEvent_t e0, e1;
    ONHIP_CHECK_HIP(hipEventCreate(&e0));
    ONHIP_CHECK_HIP(hipEventCreate(&e1));
    Choice best = guess;
    float best_ms = 1e30f, guess_ms = 1e30f;
    int rc = ONHIP_OK;
    // The model's own choice is measured first (it need not be among the candidates below), and another one takes its
    // place only by beating it by 2 %: the measurements repeat within about 3 %, and without the margin a launch that is
    // no faster replaces the model's on a coin toss (seen as a tuned stack slower than the untuned one).
    rc = time_choice(cfg, p, guess, st, e0, e1, &guess_ms);
    best_ms = guess_ms;
    auto same = [](const Choice &a, const Choice &b) {
        return a.bm == b.bm && a.bn == b.bn && a.split == b.split && a.tail == b.tail && a.rowb == b.rowb && a.fin == b.fin && a.dma == b.dma;
    };
    auto try_choice = [&](const Choice &c) {
        if (same(c, guess)) return;
        float ms = 0.f;
        rc = time_choice(cfg, p, c, st, e0, e1, &ms);
        if (!rc && ms < best_ms && ms < 0.98f * guess_ms) { best_ms = ms; best = c; }
    };
    for (int t = 0; t < kNumTiles && !rc; ++t) {
        for (int s = 0; s < kNumSplits && !rc; ++s) {
            const Choice c = {kTiles[t][0], kTiles[t][1], kSplits[s], 0, 0, 0};
            if (!candidate_ok(cfg, p, c) || model_cost(cfg, p, c) > 2.5 * guess_cost) continue;
            try_choice(c);
            const Choice cf = {c.bm, c.bn, c.split, 0, 0, 1};   // the same with the reduction inside the launch
            if (!rc && candidate_ok(cfg, p, cf)) try_choice(cf);
        }
        // the leftover column blocks as a K-split launch of about one workgroup per CU, and half as many
        int dpc = 0, left = 0;
        if (!rc && tail_geometry(cfg, p, kTiles[t][0], kTiles[t][1], &dpc, &left)) {
            int want = 256 / left;
            want = want > 16 ? 16 : want;
            for (int ts = want; ts >= 2 && ts >= want / 2 && !rc; ts /= 2) {
                const Choice c = {kTiles[t][0], kTiles[t][1], 1, ts, 0, 0};
                if (candidate_ok(cfg, p, c) && model_cost(cfg, p, {c.bm, c.bn, 1, 0, 0, 0}) <= 2.5 * guess_cost) {
                    try_choice(c);
                    const Choice cf = {c.bm, c.bn, 1, ts, 0, 1};
                    if (!rc && candidate_ok(cfg, p, cf)) try_choice(cf);
                }
            }
        }
    }
    // the kernel without LDS for B, where the problem allows it
    for (int t = 0; t < kNumRowbTiles && !rc; ++t) {
        if (kRowbTiles[t][0] == 32 && p.M > 32) continue;   // one row tile of up to 32 output channels
        if (kRowbTiles[t][0] == 96 && p.M % 96 > 0 && p.M % 96 <= 64) continue;   // a last row tile that a 64-row tile covers as well
        const Choice c = {kRowbTiles[t][0], kRowbTiles[t][1], 1, 0, 1, 0};
        if (!candidate_ok(cfg, p, c)) continue;
        try_choice(c);
        int dpc = 0, left = 0;
        if (!rc && tail_geometry(cfg, p, c.bm, c.bn, &dpc, &left)) {
            int want = 256 / left;
            want = want > 16 ? 16 : want;
            for (int ts = want; ts >= 2 && ts >= want / 2 && !rc; ts /= 2) {
                const Choice ct = {c.bm, c.bn, 1, ts, 1, 0};
                if (candidate_ok(cfg, p, ct)) try_choice(ct);
            }
        }
    }
    // the int8 kernel that loads its tiles straight into LDS
    static const int kDmaTiles[][2] = {{128, 128}, {128, 64}, {64, 128}, {64, 64}};
    for (int t = 0; t < 8 && !rc; ++t) {
        const Choice c = {kDmaTiles[t % 4][0], kDmaTiles[t % 4][1], 1, 0, 0, 0, 1 + t / 4};   // both ring lengths
        if (candidate_ok(cfg, p, c)) try_choice(c);
    }
    (void) hipEventDestroy(e0);
    (void) hipEventDestroy(e1);
    if (rc) return rc;
    if (getenv("ONHIP_TUNE_VERBOSE"))
        fprintf(stderr, "[onenew_hip] tuned dt=%d bl=%d M=%d N=%d K=%d batch=%d -> %dx%d split %d tail %d rowb %d fin %d dma %d (%.4f ms; model said %dx%d split %d dma %d)\n",
                cfg.dtype, cfg.bl, p.M, p.N, p.K, cfg.batch, best.bm, best.bn, best.split, best.tail, best.rowb, best.fin, best.dma, best_ms, guess.bm,
                guess.bn, guess.split, guess.dma);
    {
        std::lock_guard<std::mutex> lock(g_tune_mu);
        g_tuned[key] = best;
        append_tune_cache_locked(key, best);
    }
    return launch_choice(cfg, p, best, st);
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
    void *ptr = nullptr;
    return noalloc_scratch(&ptr);   // this device's address of the built-in scratch array, for onhip_conv2d_f32_noalloc
}

int onhip_set_tuning(int mode) {
    std::lock_guard<std::mutex> lock(g_tune_mu);
    const int prev = tune_mode();
    g_tune_mode = mode > 0 ? 1 : 0;
    return prev;
}

int onhip_set_tile_hint(int32_t bm, int32_t bn) {
    const Choice c = {bm, bn, 1, 0, 0, 0};
    if (bm > 0 && bn > 0 && tile_exists(c)) {
        tl_hint_bm = bm; tl_hint_bn = bn;
        return 1;
    }
    tl_hint_bm = tl_hint_bn = 0;
    return 0;
}

int onhip_tile_candidate(int32_t idx, int32_t *bm, int32_t *bn) {
    if (idx < 0 || idx >= kNumTiles || !bm || !bn) return set_error(ONHIP_ERR_ARG, "tile candidate: index %d of %d", idx, kNumTiles);
    *bm = kTiles[idx][0]; *bn = kTiles[idx][1];
    return ONHIP_OK;
}

long long onhip_scratch_bytes(void) {
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    return (long long) g_scratch_bytes;
}

long long onhip_direct_lds_launches(void) { return g_dma_launches.load(std::memory_order_relaxed); }

long long onhip_split_tail_launches(void) { return g_tail_launches.load(std::memory_order_relaxed); }

void onhip_last_launch_choice(int32_t out[7]) {
    for (int i = 0; i < 7; ++i) out[i] = tl_last_choice[i];
}

long long onhip_noalloc_scratch_launches(void) { return g_noalloc_scratch_uses.load(std::memory_order_relaxed); }

int onhip_conv_out_shape(const onhip_conv_desc_t *d, int32_t *oh, int32_t *ow) {
    if (!oh || !ow) return set_error(ONHIP_ERR_ARG, "conv: null output pointer");
    return check_conv(d, oh, ow);
}

// channels per filter tap in the tap-major packed weight layout (padded to whole MFMA units)
static int packed_cp(const onhip_conv_desc_t *d) {
    const int kpu = d->compute == ONHIP_COMPUTE_F32 ? 4 : 8;
    return (d->cin + kpu - 1) / kpu * kpu;
}

// Dense convolutions other than the plain 1x1 have a packed weight form: the first-layer kernel's own, or the tap-major one.
// Not the tap-major one where it would cost more than it saves: fewer than four input channels (a tap is padded to four:
// a third more reduction) and filters of more than 64 taps (validity by coordinates instead of the lane's mask); the
// element gather on the weights as they are measures 25 % ahead there (ViT's 16 x 16 patch convolution: 63 against 83 us).
// a 1x1 filter without padding: the input itself is the B operand, no window arithmetic
static bool plain_pointwise(const onhip_conv_desc_t *d) {
    return d->kh == 1 && d->kw == 1 && !d->pad_t && !d->pad_l && !d->pad_b && !d->pad_r;
}
static bool wants_packed(const onhip_conv_desc_t *d) {
    if (d->group != 1 || plain_pointwise(d)) return false;
    return stem_f32_shape(*d) || (d->cin >= 4 && d->kh * d->kw <= 64);
}

size_t onhip_conv2d_packed_weight_bytes(const onhip_conv_desc_t *d) {
    if (!d || d->cin < 1 || d->cout < 1 || d->kh < 1 || d->kw < 1 || !wants_packed(d)) return 0;
    if (stem_f32_shape(*d)) return (size_t) ((d->kh * d->kw * 3 + 1) / 2 * 2) * 64 * sizeof(float);   // [reduction index][64]
    return (size_t) d->cout * d->kh * d->kw * packed_cp(d) * sizeof(float);
}

int onhip_conv2d_pack_weights(const onhip_conv_desc_t *d, const float *w, float *packed, void *stream) {
    int32_t OH, OW;
    int rc = check_conv(d, &OH, &OW);
    if (rc) return rc;
    if (!w || !packed) return set_error(ONHIP_ERR_ARG, "conv pack: null pointer");
    if (!wants_packed(d)) return set_error(ONHIP_ERR_ARG, "conv pack: this convolution takes its weights as they are");
    // a first-layer convolution (three input channels): the layout of the kernel that runs it, whatever the image size
    if (stem_f32_shape(*d)) return stem_pack_launch(*d, w, packed, reinterpret_cast<hipStream_t>(stream));
    return pack_wf32_launch(w, d->cout, d->cin, d->kh * d->kw, packed_cp(d), packed, reinterpret_cast<hipStream_t>(stream));
}

// packed != 0: w holds the tap-major layout written by onhip_conv2d_pack_weights
// the Add (and Relu) of a residual block as separate passes over y, for the paths whose store cannot fold them in
static int add_relu_in_place(const onhip_conv_desc_t *d, int OH, int OW, const float *addend, int relu, float *y, void *stream) {
    onhip_add_desc_t ad;
    memset(&ad, 0, sizeof(ad));
    ad.ndim = 4;
    const int32_t shape[4] = {d->n, d->cout, OH, OW};
    for (int i = 0; i < 4; ++i) ad.large_shape[i] = ad.small_shape[i] = shape[i];
    int rc = onhip_add_f32(&ad, y, addend, y, stream);
    if (!rc && relu) rc = onhip_relu_f32(y, y, (long long) d->n * d->cout * OH * OW, stream);
    return rc;
}

static int conv2d_f32_impl(const onhip_conv_desc_t *d, const float *x, const float *w, int packed, const float *bias,
                           const float *silu_lut, float *y, void *stream, const float *addend = nullptr, int relu_after = 0) {
    int32_t OH, OW;
    int rc = check_conv(d, &OH, &OW);
    if (rc) return rc;
    if (!x || !w || !y || (d->has_bias && !bias)) return set_error(ONHIP_ERR_ARG, "conv: null tensor pointer");
    if (addend == y) return set_error(ONHIP_ERR_ARG, "conv: the addend may not be the output buffer");
    if (d->has_bias && d->act_type == SILU && !silu_lut) return set_error(ONHIP_ERR_ARG, "conv: SILU needs the table");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const Epilogue ep = make_epilogue(*d, silu_lut);
    if (packed && !wants_packed(d)) return set_error(ONHIP_ERR_ARG, "conv: this convolution has no packed weight form");
    if (d->group != 1) {
        if (d->compute != ONHIP_COMPUTE_F32)
            return set_error(ONHIP_ERR_ARG, "conv: depthwise runs in fp32 only");
        rc = depthwise_f32_launch(*d, OH, OW, x, w, bias, ep, y, st);
        if (!rc && addend) rc = add_relu_in_place(d, OH, OW, addend, relu_after, y, stream);
        return rc;
    }
    // First-layer convolutions: packed weights have that kernel's layout, so it runs them whatever the image size (and
    // the Add of a residual block, which no first layer has, as a pass of its own); weights as given only where rows of
    // 96 pixels and more fill its workgroups.
    static const bool no_stem = getenv("ONHIP_NO_STEM") != nullptr;   // tuning hook: unpacked weights on the implicit-GEMM kernels
    if (stem_f32_ok(*d, OH, OW) && (packed || (OW >= 96 && !addend && !no_stem))) {
        rc = stem_f32_launch(*d, OH, OW, x, w, packed, bias, ep, y, st);
        if (!rc && addend) rc = add_relu_in_place(d, OH, OW, addend, relu_after, y, stream);
        return rc;
    }
    if (packed && stem_f32_shape(*d)) return set_error(ONHIP_ERR_ARG, "conv: first-layer tensors of 2^29 elements or more are not supported with packed weights");
    IgemmLaunch cfg;
    memset(&cfg, 0, sizeof(cfg));
    rc = dtype_of_compute(d->compute, &cfg.dtype);
    if (rc) return rc;
    cfg.batch = 1;
    IgemmParams p;
    memset(&p, 0, sizeof(p));
    const int kpu = kpu_of(cfg.dtype);
    p.M = d->cout;
    p.N = d->n * OH * OW;
    p.H = d->h; p.W = d->w; p.OW = OW; p.OHW = OH * OW; p.HW = d->h * d->w;
    p.kh = d->kh; p.kw = d->kw; p.khkw = d->kh * d->kw;
    p.sh = d->stride_h; p.sw = d->stride_w; p.pt = d->pad_t; p.pl = d->pad_l;
    p.magic_khkw = magic_for(p.khkw); p.pass_khkw = pass_for(p.khkw);
    p.magic_kw = magic_for(p.kw); p.pass_kw = pass_for(p.kw);
    p.use_tapmask = p.khkw <= 64;
    if (packed) {
        // K = (tap, channel): every unit of KPU channels shares one filter tap
        const int cp = packed_cp(d);
        cfg.bl = BL_TAPC;
        p.K = p.khkw * cp;
        p.units_per_tap = cp / kpu;
        p.magic_upt = magic_for(p.units_per_tap); p.pass_upt = pass_for(p.units_per_tap);
    } else {
        cfg.bl = plain_pointwise(d) ? BL_PLAIN : BL_GATHER;
        p.K = d->cin * p.khkw;
    }
    if ((unsigned long long) p.K * (unsigned) p.khkw >= (1ULL << 32))
        return set_error(ONHIP_ERR_ARG, "conv: reduction length %d too large", p.K);
    p.k_units = (p.K + kpu - 1) / kpu;
    p.A = w;
    p.lda = p.K;
    p.B = x;
    p.b_img_stride = (long long) d->cin * d->h * d->w;
    p.b_shift_bytes = ((long long) d->pad_t * d->w + d->pad_l) * 4;
    p.a_slice_bytes = (long long) p.M * p.K * 4;
    p.b_slice_bytes = (long long) d->n * p.b_img_stride * 4;
    p.c_slice_bytes = (long long) d->n * d->cout * OH * OW * 4;
    p.C = y;
    p.out_mode = OUT_CONV;
    p.c_img_stride = (long long) d->cout * OH * OW;
    p.c_stride_m = (long long) OH * OW;
    p.bias = bias;
    p.bias_mode = d->has_bias ? BIAS_M : BIAS_NONE;
    p.ep = ep;
    if (addend && cfg.dtype != DT_F32) {   // reduced-precision operands: the two operators as passes over y
        rc = plan_and_launch(cfg, p, st);
        if (!rc) rc = add_relu_in_place(d, OH, OW, addend, relu_after, y, stream);
        return rc;
    }
    if (addend) {
        const long long n_out = (long long) d->n * d->cout * OH * OW;
        p.res = addend;
        p.res_relu = relu_after ? 1 : 0;
        p.res_body = (unsigned) (n_out - n_out % 32);   // relu.c:27-52
    }
    return plan_and_launch(cfg, p, st);
}

int onhip_conv2d_f32_add(const onhip_conv_desc_t *d, const float *x, const float *w, int32_t packed, const float *bias,
                         const float *silu_lut, const float *addend, int32_t relu_after, float *y, void *stream) {
    if (!addend) return set_error(ONHIP_ERR_ARG, "conv + add: null addend");
    return conv2d_f32_impl(d, x, w, packed ? 1 : 0, bias, silu_lut, y, stream, addend, relu_after);
}

int onhip_conv2d_f32(const onhip_conv_desc_t *d, const float *x, const float *w, const float *bias,
                     const float *silu_lut, float *y, void *stream) {
    return conv2d_f32_impl(d, x, w, 0, bias, silu_lut, y, stream);
}

int onhip_conv2d_f32_packed(const onhip_conv_desc_t *d, const float *x, const float *w_packed, const float *bias,
                            const float *silu_lut, float *y, void *stream) {
    return conv2d_f32_impl(d, x, w_packed, 1, bias, silu_lut, y, stream);
}

int onhip_conv2d_f32_noalloc(const onhip_conv_desc_t *d, const float *x, const float *w, int32_t packed, const float *bias,
                             const float *silu_lut, float *y, void *stream) {
    void *ptr = nullptr;
    int rc = noalloc_scratch(&ptr);   // a lookup on the first call on a device (onhip_init has done it already), no allocation
    if (rc) return rc;
    tl_noalloc = ptr;
    rc = conv2d_f32_impl(d, x, w, packed ? 1 : 0, bias, silu_lut, y, stream);
    tl_noalloc = nullptr;
    return rc;
}

// ---- a convolution and the 1x1 convolution after it in one launch ------------------------------------------------------------
static bool act_none_relu_clip(int act) { return act == NOT_ACT || act == RELU6 || act == RELU || act == CLIP; }

// what the pair must look like; *why names the first condition that fails
static bool conv_pw_shapes_ok(const onhip_conv_desc_t *a, const onhip_conv_desc_t *b, int OH, int OW, const char **why) {
    *why = nullptr;
    if (a->compute != ONHIP_COMPUTE_F32 || b->compute != ONHIP_COMPUTE_F32) *why = "fp32 only";
    else if (a->group != 1 || b->group != 1) *why = "dense convolutions only";
    else if (!wants_packed(a) || stem_f32_shape(*a)) *why = "the first convolution must be one that takes tap-major packed weights";
    else if (a->cout > 64) *why = "the first convolution must have at most 64 output channels";
    else if (b->kh != 1 || b->kw != 1 || b->stride_h != 1 || b->stride_w != 1 || b->pad_t || b->pad_l || b->pad_b || b->pad_r)
        *why = "the second convolution must be 1x1, stride 1, without padding";
    else if (b->cin != a->cout || b->n != a->n || b->h != OH || b->w != OW) *why = "the second convolution does not read the first one's result";
    else if (!act_none_relu_clip(a->act_type) || !act_none_relu_clip(b->act_type)) *why = "activations other than none, Relu and Clip";
    else if (a->kh * a->kw > 64) *why = "filters of more than 64 taps";
    else if ((long long) a->n * b->cout * OH * OW >= (1LL << 29) || (long long) a->n * a->cin * a->h * a->w >= (1LL << 29))
        *why = "tensors of 2^29 elements or more";
    return *why == nullptr;
}

int onhip_conv2d_pw_supported(const onhip_conv_desc_t *a, const onhip_conv_desc_t *b) {
    int32_t OH, OW, OH2, OW2;
    if (check_conv(a, &OH, &OW) || check_conv(b, &OH2, &OW2)) return 0;
    const char *why;
    if (!conv_pw_shapes_ok(a, b, OH, OW, &why)) return 0;
    // expected to pay: the first result is wide in pixels and narrow in channels, so that writing and re-reading it
    // and a launch of its own cost more than the occupancy its registers take from the first product
    return (long long) a->n * OH * OW >= 16384 ? 2 : 1;
}

size_t onhip_conv2d_pw_packed_weight_bytes(const onhip_conv_desc_t *b) {
    if (!b || b->cout < 1 || b->cin < 1 || b->cin > 64) return 0;
    return (size_t) ((b->cout + 63) / 64) * 64 * 64 * sizeof(float);
}

int onhip_conv2d_pw_pack_weights(const onhip_conv_desc_t *b, const float *wb, float *packed, void *stream) {
    if (!onhip_conv2d_pw_packed_weight_bytes(b)) return set_error(ONHIP_ERR_ARG, "conv + 1x1 pack: a 1x1 convolution over at most 64 channels");
    if (!wb || !packed || reinterpret_cast<uintptr_t>(packed) % 16) return set_error(ONHIP_ERR_ARG, "conv + 1x1 pack: null or unaligned pointer");
    return pack_pw2_launch(wb, b->cout, b->cin, packed, reinterpret_cast<hipStream_t>(stream));
}

int onhip_conv2d_pw_f32(const onhip_conv_desc_t *a, const onhip_conv_desc_t *b, const float *x, const float *wa_packed,
                        const float *bias_a, const float *wb_packed, const float *bias_b, const float *addend, int32_t relu_after,
                        float *y, void *stream) {
    int32_t OH, OW, OH2, OW2;
    int rc = check_conv(a, &OH, &OW);
    if (!rc) rc = check_conv(b, &OH2, &OW2);
    if (rc) return rc;
    const char *why;
    if (!conv_pw_shapes_ok(a, b, OH, OW, &why)) return set_error(ONHIP_ERR_ARG, "conv + 1x1: %s", why);
    if (!x || !wa_packed || !wb_packed || !y || (a->has_bias && !bias_a) || (b->has_bias && !bias_b))
        return set_error(ONHIP_ERR_ARG, "conv + 1x1: null tensor pointer");
    if (addend == y) return set_error(ONHIP_ERR_ARG, "conv + 1x1: the addend may not be the output buffer");
    IgemmParams p;
    memset(&p, 0, sizeof(p));
    const int cp = packed_cp(a);
    p.M = a->cout;
    p.N = a->n * OH * OW;
    p.H = a->h; p.W = a->w; p.OW = OW; p.OHW = OH * OW; p.HW = a->h * a->w;
    p.kh = a->kh; p.kw = a->kw; p.khkw = a->kh * a->kw;
    p.sh = a->stride_h; p.sw = a->stride_w; p.pt = a->pad_t; p.pl = a->pad_l;
    p.magic_khkw = magic_for(p.khkw); p.pass_khkw = pass_for(p.khkw);
    p.magic_kw = magic_for(p.kw); p.pass_kw = pass_for(p.kw);
    p.use_tapmask = 1;
    p.K = p.khkw * cp;
    p.units_per_tap = cp / 4;
    p.magic_upt = magic_for(p.units_per_tap); p.pass_upt = pass_for(p.units_per_tap);
    p.k_units = p.K / 4;
    p.A = wa_packed;
    p.lda = p.K;
    p.B = x;
    p.b_img_stride = (long long) a->cin * a->h * a->w;
    p.b_shift_bytes = ((long long) a->pad_t * a->w + a->pad_l) * 4;
    p.a_slice_bytes = (long long) p.M * p.K * 4;
    p.b_slice_bytes = (long long) a->n * p.b_img_stride * 4;
    p.c_slice_bytes = (long long) a->n * b->cout * OH * OW * 4;
    p.C = y;
    p.out_mode = OUT_CONV;
    p.c_img_stride = (long long) b->cout * OH * OW;
    p.c_stride_m = (long long) OH * OW;
    p.bias = bias_a;
    p.bias_mode = a->has_bias ? BIAS_M : BIAS_NONE;
    p.ep = make_epilogue(*a, nullptr);
    p.w2 = wb_packed;
    p.bias2 = b->has_bias ? bias_b : nullptr;
    p.m2 = b->cout;
    p.ep2 = make_epilogue(*b, nullptr);
    if (addend) {
        const long long n_out = (long long) a->n * b->cout * OH * OW;
        p.res = addend;
        p.res_relu = relu_after ? 1 : 0;
        p.res_body = (unsigned) (n_out - n_out % 32);   // relu.c:27-52
    }
    return igemm_launch_f32_pw(p, reinterpret_cast<hipStream_t>(stream));
}

static void w8a32_layout(const onhip_conv_desc_t *d, int *cp, int *k_units, size_t *packed_bytes, size_t *q_bytes) {
    *cp = (d->cin + 15) / 16 * 16;
    *k_units = d->kh * d->kw * (*cp / 16);
    *packed_bytes = ((size_t) d->cout * *k_units * 16 + 255) / 256 * 256;
    *q_bytes = ((size_t) d->n * d->h * d->w * *cp + 255) / 256 * 256;
}

size_t onhip_conv2d_w8a32_workspace(const onhip_conv_desc_t *d) {
    if (!d) return 0;
    int cp, ku;
    size_t pb, qb;
    w8a32_layout(d, &cp, &ku, &pb, &qb);
    // depthwise: only the form with fp32 activations in and an int8 NHWC result out stages anything (the quantised input)
    return d->group != 1 ? qb : pb + qb;
}

size_t onhip_conv2d_w8a32_packed_weight_bytes(const onhip_conv_desc_t *d) {
    if (!d || d->group != 1 || d->cin < 1 || d->cout < 1 || d->kh < 1 || d->kw < 1) return 0;
    int cp, ku;
    size_t pb, qb;
    w8a32_layout(d, &cp, &ku, &pb, &qb);
    return pb;
}

int onhip_conv2d_w8a32_pack_weights(const onhip_conv_desc_t *d, const int8_t *w8, int8_t *packed, void *stream) {
    int32_t OH, OW;
    int rc = check_conv(d, &OH, &OW);
    if (rc) return rc;
    if (!w8 || !packed) return set_error(ONHIP_ERR_ARG, "conv w8a32 pack: null pointer");
    if (d->group != 1) return set_error(ONHIP_ERR_ARG, "conv w8a32 pack: depthwise weights are used as they are");
    int cp, k_units;
    size_t pb, qb;
    w8a32_layout(d, &cp, &k_units, &pb, &qb);
    return pack_w8_launch(w8, d->cout, d->cin, d->kh, d->kw, cp, k_units, packed, reinterpret_cast<hipStream_t>(stream));
}

// packed != 0: w8 holds the layout written by onhip_conv2d_w8a32_pack_weights and the workspace only
// takes the int8 copy of the activations
// Tables that have been through an output quantiser, by (table address, 1 / output scale): built on first use on the
// caller's stream and kept for the life of the process.  The activation tables are constants of the model runtime
// (host/ops/conv.h:178-194 builds one per process); a caller that rewrites one in place gets the old bytes.
static std::mutex g_qlut_mu;
static std::map<std::pair<const float *, uint32_t>, signed char *> g_qlut;

static int quantised_table(const float *lut, float out_inv_scale, hipStream_t st, const signed char **out) {
    uint32_t bits;
    memcpy(&bits, &out_inv_scale, 4);
    std::lock_guard<std::mutex> lock(g_qlut_mu);
    auto key = std::make_pair(lut, bits);
    auto it = g_qlut.find(key);
    if (it == g_qlut.end()) {
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
            *out = nullptr;   // no allocation while a graph is being recorded: the float table serves
            return ONHIP_OK;
        }
        signed char *q = nullptr;
        ONHIP_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&q), 8192));
        int rc = build_qlut_launch(lut, out_inv_scale, q, st);
        if (rc) { (void) hipFree(q); return rc; }
        it = g_qlut.emplace(key, q).first;
    }
    *out = it->second;
    return ONHIP_OK;
}

// Drops the quantised copies of tables whose address lies in [base, base + bytes): that memory is about to be freed or
// rewritten, and another table at the same address must be quantised afresh.
extern "C++" {
int onhip::forget_quantised_tables(const void *base, size_t bytes) {
    std::lock_guard<std::mutex> lock(g_qlut_mu);
    const char *lo = static_cast<const char *>(base), *hi = lo + bytes;
    bool any = false;
    for (auto it = g_qlut.begin(); it != g_qlut.end();) {
        const char *k = reinterpret_cast<const char *>(it->first.first);
        if (k >= lo && k < hi) {
            if (!any) ONHIP_CHECK_HIP(hipDeviceSynchronize());   // a kernel may still be reading the copy
            any = true;
            (void) hipFree(it->second);
            it = g_qlut.erase(it);
        } else {
            ++it;
        }
    }
    return ONHIP_OK;
}
}   // extern "C++"

// xq != nullptr: the activations arrive already quantised (int8 NHWC, channels padded to 16) and x is not read;
// nhwc_out != 0: the int8 result is written NHWC with its channels padded to 16, ready to be the next xq
static int conv2d_w8a32_impl(const onhip_conv_desc_t *d, const float *x, const int8_t *xq, const int8_t *w8, int packed_w,
                             const int32_t *bias32, const float *weight_aux, const float *silu_lut, void *y,
                             int32_t *acc32, void *workspace, size_t workspace_bytes, int nhwc_out, void *stream,
                             const float *addend = nullptr, int relu_after = 0, int8_t *twin = nullptr) {
    int32_t OH, OW;
    int rc = check_conv(d, &OH, &OW);
    if (rc) return rc;
    if ((!x && !xq) || !w8 || !y || !weight_aux || (d->has_bias && !bias32))
        return set_error(ONHIP_ERR_ARG, "conv w8a32: null tensor pointer");
    if (nhwc_out && !d->out_s8) return set_error(ONHIP_ERR_ARG, "conv w8a8: the NHWC output form is int8 (out_s8 = 1)");
    if (addend && (d->out_s8 || acc32 || d->group != 1))
        return set_error(ONHIP_ERR_ARG, "conv w8a32: an addend goes with dense convolutions and fp32 results");
    if (twin && (!addend || d->cout % 16 || !(d->output_scale > 0.0f) || reinterpret_cast<uintptr_t>(twin) % 4 ||
                 (long long) d->n * OH * OW * d->cout >= (1LL << 31)))
        return set_error(ONHIP_ERR_ARG, "conv w8a32: the int8 twin goes with an addend, output channels in sixteens and an output_scale");
    // the reference pads all four sides by pads[0] (conv.c:979-999) while shapes come from the four
    // pads: only uniform padding is self-consistent
    if (d->pad_t != d->pad_l || d->pad_t != d->pad_b || d->pad_t != d->pad_r)
        return set_error(ONHIP_ERR_ARG, "conv w8a32: padding must be uniform");
    if (!(d->input_scale > 0.0f)) return set_error(ONHIP_ERR_ARG, "conv w8a32: input_scale must be positive");
    if (d->out_s8 && !(d->output_scale > 0.0f)) return set_error(ONHIP_ERR_ARG, "conv w8a32: output_scale must be positive");
    if (d->has_bias && d->act_type == SILU && !silu_lut) return set_error(ONHIP_ERR_ARG, "conv: SILU needs the table");
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const Epilogue ep = make_epilogue(*d, silu_lut);
    if (d->group != 1) {
        // depthwise weights have no packed form: every entry point takes them as the reference holds them
        if (!xq && !nhwc_out) return depthwise_w8a32_launch(*d, OH, OW, x, w8, bias32, weight_aux, ep, y, acc32, st);
        // an int8 NHWC tensor on either side: the kernel of the chain form.  fp32 activations are quantised into the
        // workspace first (the staging pass of the dense W8A32 form); an fp32 result is written NCHW by the kernel
        if (acc32) return set_error(ONHIP_ERR_ARG, "conv w8a8: depthwise accumulators are available in the fp32 form only");
        if (!dw_s8_ok(*d, OH, OW)) return set_error(ONHIP_ERR_ARG, "conv w8a8: depthwise with %d channels and a %dx%d filter is not available in the NHWC int8 form", d->cout, d->kh, d->kw);
        const int cpd = (d->cin + 15) / 16 * 16;
        const int8_t *q8 = xq;
        if (!xq) {
            const size_t need = (size_t) d->n * d->h * d->w * cpd;
            if (!workspace || workspace_bytes < need || reinterpret_cast<uintptr_t>(workspace) % 16)
                return set_error(ONHIP_ERR_WORKSPACE, "conv w8a8: depthwise needs a 16-byte aligned workspace of %zu bytes for the quantised input, %zu given",
                                 need, workspace ? workspace_bytes : (size_t) 0);
            rc = quantize_nhwc_launch(x, d->n, d->cin, d->h, d->w, cpd, 1.0f / d->input_scale, reinterpret_cast<int8_t *>(workspace), st);
            if (rc) return rc;
            q8 = reinterpret_cast<const int8_t *>(workspace);
        } else if (reinterpret_cast<uintptr_t>(xq) % 16) {
            return set_error(ONHIP_ERR_ARG, "conv w8a8: int8 activations must be 16-byte aligned");
        }
        if (nhwc_out && reinterpret_cast<uintptr_t>(y) % 16) return set_error(ONHIP_ERR_ARG, "conv w8a8: the int8 result must be 16-byte aligned");
        return dw_s8_launch(*d, OH, OW, q8, w8, bias32, weight_aux, ep, y, st);
    }

    int cp, k_units;
    size_t packed_bytes, q_bytes;
    w8a32_layout(d, &cp, &k_units, &packed_bytes, &q_bytes);
    if (packed_w) packed_bytes = 0;
    if (xq) q_bytes = 0;
    if (packed_bytes + q_bytes > 0 && (!workspace || workspace_bytes < packed_bytes + q_bytes))
        return set_error(ONHIP_ERR_WORKSPACE, "conv w8a32: workspace of %zu bytes needed, %zu given",
                         packed_bytes + q_bytes, workspace ? workspace_bytes : (size_t) 0);
    if (packed_bytes + q_bytes > 0 && reinterpret_cast<uintptr_t>(workspace) % 16)
        return set_error(ONHIP_ERR_WORKSPACE, "conv w8a32: workspace must be 16-byte aligned");
    if (xq && reinterpret_cast<uintptr_t>(xq) % 16)
        return set_error(ONHIP_ERR_ARG, "conv w8a8: int8 activations must be 16-byte aligned");
    if ((long long) d->n * d->h * d->w * cp >= (1LL << 31))
        return set_error(ONHIP_ERR_ARG, "conv w8a32: staged activations of 2 GiB or more are not supported");
    const int8_t *packed = w8;
    int8_t *q = reinterpret_cast<int8_t *>(workspace) + packed_bytes;
    if (!packed_w) {
        int8_t *dst = reinterpret_cast<int8_t *>(workspace);
        rc = pack_w8_launch(w8, d->cout, d->cin, d->kh, d->kw, cp, k_units, dst, st);
        if (rc) return rc;
        packed = dst;
    } else if (reinterpret_cast<uintptr_t>(w8) % 16) {
        return set_error(ONHIP_ERR_ARG, "conv w8a32: packed weights must be 16-byte aligned");
    }
    if (xq) {
        q = const_cast<int8_t *>(xq);
    } else {
        rc = quantize_nhwc_launch(x, d->n, d->cin, d->h, d->w, cp, 1.0f / d->input_scale, q, st);
        if (rc) return rc;
    }

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
    p.use_tapmask = p.khkw <= 64;
    p.units_per_tap = cp / 16;
    p.magic_upt = magic_for(p.units_per_tap); p.pass_upt = pass_for(p.units_per_tap);
    // K tiles (4 units) inside one filter tap: the loader variant with scalar tap arithmetic
    if (p.use_tapmask && p.units_per_tap % 4 == 0) cfg.bl = BL_KVEC_TAP;
    p.pix_stride = cp;
    p.b_shift_bytes = ((long long) d->pad_t * d->w + d->pad_l) * cp;
    p.a_slice_bytes = (long long) p.M * p.lda;
    p.b_slice_bytes = (long long) d->n * d->h * d->w * cp;
    p.c_slice_bytes = (long long) d->n * d->cout * OH * OW * 4;
    p.C = y;
    if (nhwc_out) {
        // element (pixel n, channel m) at n * Cp_out + m
        p.out_mode = OUT_PLAIN;
        p.c_stride_m = 1;
        p.c_stride_n = (d->cout + 15) / 16 * 16;
    } else {
        p.out_mode = OUT_CONV;
        p.c_img_stride = (long long) d->cout * OH * OW;
        p.c_stride_m = (long long) OH * OW;
    }
    p.ep = ep;
    p.in_scale = d->input_scale;
    p.weight_aux = weight_aux;
    p.bias32 = d->has_bias ? bias32 : nullptr;
    p.acc_out = acc32;
    p.out_s8 = d->out_s8;
    p.out_inv_scale = d->out_s8 ? 1.0f / d->output_scale : 0.0f;
    if (nhwc_out && ep.act == SILU && ep.lut && !acc32) {   // the staged int8 store: gather quantised table entries
        rc = quantised_table(ep.lut, p.out_inv_scale, st, &p.ep.qlut);
        if (rc) return rc;
    }
    if (addend) {   // the Add (and Relu) after the convolution, in its store
        const long long n_out = (long long) d->n * d->cout * OH * OW;
        p.res = addend;
        p.res_relu = relu_after ? 1 : 0;
        p.res_body = (unsigned) (n_out - n_out % 32);   // relu.c:27-52
        p.twin = twin;
        p.twin_pitch = d->cout;
        p.twin_inv_scale = twin ? 1.0f / d->output_scale : 0.0f;
    }
    // 3x3, stride 1, few channels, int8 in and out: the kernel that keeps the band's input in LDS and the weights in registers
    // tuning hooks: ONHIP_NO_PATCH keeps to the implicit-GEMM kernels, and so does a forced tile of theirs; ONHIP_PATCH_ALL
    // sends every shape the LDS-patch kernel can take to it, not only those it is measured to win
    const bool no_patch = getenv("ONHIP_NO_PATCH") != nullptr || getenv("ONHIP_TILE") != nullptr;
    if (nhwc_out && !no_patch && i8patch_ok(p, getenv("ONHIP_PATCH_ALL") != nullptr)) return i8patch_launch(p, st);
    if (nhwc_out && !no_patch && i8direct_ok(p)) return i8direct_launch(p, st);
    return plan_and_launch(cfg, p, st);
}

int onhip_conv2d_w8a32(const onhip_conv_desc_t *d, const float *x, const int8_t *w8, const int32_t *bias32,
                       const float *weight_aux, const float *silu_lut, void *y, int32_t *acc32, void *workspace,
                       size_t workspace_bytes, void *stream) {
    return conv2d_w8a32_impl(d, x, nullptr, w8, 0, bias32, weight_aux, silu_lut, y, acc32, workspace, workspace_bytes, 0, stream);
}

int onhip_conv2d_w8a32_packed(const onhip_conv_desc_t *d, const float *x, const int8_t *w8_packed,
                              const int32_t *bias32, const float *weight_aux, const float *silu_lut, void *y,
                              int32_t *acc32, void *workspace, size_t workspace_bytes, void *stream) {
    return conv2d_w8a32_impl(d, x, nullptr, w8_packed, 1, bias32, weight_aux, silu_lut, y, acc32, workspace, workspace_bytes,
                             0, stream);
}

int onhip_quantize_nhwc_s8(const float *x, int32_t n, int32_t c, int32_t h, int32_t w, float scale, int8_t *q, void *stream) {
    if (!x || !q || n < 1 || c < 1 || h < 1 || w < 1 || !(scale > 0.0f)) return set_error(ONHIP_ERR_ARG, "quantize: bad argument");
    const int cp = (c + 15) / 16 * 16;
    if ((long long) n * h * w * cp >= (1LL << 31)) return set_error(ONHIP_ERR_ARG, "quantize: tensor too large");
    if (reinterpret_cast<uintptr_t>(q) % 16) return set_error(ONHIP_ERR_ARG, "quantize: output must be 16-byte aligned");
    return quantize_nhwc_launch(x, n, c, h, w, cp, 1.0f / scale, q, reinterpret_cast<hipStream_t>(stream));
}

int onhip_conv2d_w8a8_nhwc(const onhip_conv_desc_t *d, const int8_t *xq, const int8_t *w8_packed, const int32_t *bias32,
                           const float *weight_aux, const float *silu_lut, int8_t *yq, void *stream) {
    if (!d) return set_error(ONHIP_ERR_ARG, "conv w8a8: null descriptor");
    onhip_conv_desc_t dd = *d;
    dd.out_s8 = 1;
    return conv2d_w8a32_impl(&dd, nullptr, xq, w8_packed, 1, bias32, weight_aux, silu_lut, yq, nullptr, nullptr, 0, 1, stream);
}

int onhip_conv2d_w8a8_depthwise_supported(const onhip_conv_desc_t *d) {
    int32_t OH = 0, OW = 0;
    if (!d || d->group == 1 || check_conv(d, &OH, &OW)) return 0;
    if (d->pad_t != d->pad_l || d->pad_t != d->pad_b || d->pad_t != d->pad_r) return 0;
    return dw_s8_ok(*d, OH, OW) ? 1 : 0;
}

int onhip_conv2d_w8_link(const onhip_conv_desc_t *d, const float *x, const int8_t *xq, const int8_t *w8_packed,
                         const int32_t *bias32, const float *weight_aux, const float *silu_lut, const float *addend,
                         int32_t relu_after, void *y, int8_t *y_twin, void *workspace, size_t workspace_bytes, void *stream) {
    if (!d) return set_error(ONHIP_ERR_ARG, "conv w8 link: null descriptor");
    if ((x != nullptr) == (xq != nullptr)) return set_error(ONHIP_ERR_ARG, "conv w8 link: exactly one of x and xq");
    return conv2d_w8a32_impl(d, x, xq, w8_packed, 1, bias32, weight_aux, silu_lut, y, nullptr, workspace, workspace_bytes,
                             d->out_s8 ? 1 : 0, stream, addend, relu_after, y_twin);
}

static int matmul_impl(const onhip_matmul_desc_t *d, const float *a, const float *b, const float *bias,
                       const float *gelu_lut, const float *addend, float *out, void *stream) {
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
    // more rows than columns: the left operand is the large one (activations against a weight matrix), so tiles are
    // numbered along N first and an XCD reads its rows of A once for all column blocks
    p.n_fast = M > d->n ? 1 : 0;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (addend == out) return set_error(ONHIP_ERR_ARG, "matmul: the addend may not be the output buffer");
    if (addend && cfg.dtype != DT_F32) {   // reduced-precision operands: the Add as a pass over the result
        rc = plan_and_launch(cfg, p, st);
        if (rc) return rc;
        onhip_add_desc_t ad;
        memset(&ad, 0, sizeof(ad));
        ad.ndim = 2;
        ad.large_shape[0] = ad.small_shape[0] = batch * M;
        ad.large_shape[1] = ad.small_shape[1] = d->n;
        return onhip_add_f32(&ad, out, addend, out, stream);
    }
    p.res = addend;   // laid out like the result; added after the bias, as the Add operator after it would
    return plan_and_launch(cfg, p, st);
}

int onhip_matmul(const onhip_matmul_desc_t *d, const float *a, const float *b, const float *bias,
                 const float *gelu_lut, float *out, void *stream) {
    return matmul_impl(d, a, b, bias, gelu_lut, nullptr, out, stream);
}

int onhip_matmul_add(const onhip_matmul_desc_t *d, const float *a, const float *b, const float *bias,
                     const float *addend, float *out, void *stream) {
    if (!addend) return set_error(ONHIP_ERR_ARG, "matmul_add: null addend");
    return matmul_impl(d, a, b, bias, nullptr, addend, out, stream);
}

// ---- 16-bit storage: bf16 / fp16 operands and results in memory, fp32 accumulation ---------------------------------------
static int h16_dtype(int compute, int *dt) {
    if (compute == ONHIP_COMPUTE_BF16) { *dt = DT_BF16; return ONHIP_OK; }
    if (compute == ONHIP_COMPUTE_F16) { *dt = DT_F16; return ONHIP_OK; }
    return set_error(ONHIP_ERR_ARG, "16-bit storage: compute type %d is neither bf16 nor fp16", compute);
}

int32_t onhip_h16_pitch(int32_t channels) { return channels < 1 ? 0 : (channels + 31) / 32 * 32; }

size_t onhip_h16_packed_weight_bytes(int32_t rows, int32_t cin, int32_t taps) {
    if (rows < 1 || cin < 1 || taps < 1) return 0;
    return (size_t) rows * taps * onhip_h16_pitch(cin) * 2;
}

int onhip_h16_pack_conv_weights(const onhip_conv_desc_t *d, const float *w, void *packed, void *stream) {
    int32_t OH, OW;
    int dt, rc = check_conv(d, &OH, &OW);
    if (rc) return rc;
    if ((rc = h16_dtype(d->compute, &dt))) return rc;
    if (d->group != 1) return set_error(ONHIP_ERR_ARG, "16-bit storage: dense convolutions only");
    if (!w || !packed || reinterpret_cast<uintptr_t>(packed) % 16) return set_error(ONHIP_ERR_ARG, "16-bit pack: null or unaligned pointer");
    const int taps = d->kh * d->kw;
    return pack_w16_launch(dt, w, d->cout, d->cin, taps, onhip_h16_pitch(d->cin), (long long) d->cin * taps, taps, 1, packed,
                           reinterpret_cast<hipStream_t>(stream));
}

int onhip_h16_pack_matmul_weights(const float *b, int32_t k, int32_t n, int32_t compute, void *packed, void *stream) {
    int dt, rc = h16_dtype(compute, &dt);
    if (rc) return rc;
    if (!b || !packed || k < 1 || n < 1 || reinterpret_cast<uintptr_t>(packed) % 16) return set_error(ONHIP_ERR_ARG, "16-bit pack: bad argument");
    return pack_w16_launch(dt, b, n, k, 1, onhip_h16_pitch(k), 1, n, 0, packed, reinterpret_cast<hipStream_t>(stream));
}

int onhip_h16_from_nchw_f32(const float *x, int32_t n, int32_t c, int32_t h, int32_t w, int32_t compute, void *y, void *stream) {
    int dt, rc = h16_dtype(compute, &dt);
    if (rc) return rc;
    if (!x || !y || n < 1 || c < 1 || h < 1 || w < 1 || reinterpret_cast<uintptr_t>(y) % 16) return set_error(ONHIP_ERR_ARG, "16-bit conversion: bad argument");
    return nchw_to_nhwc16_launch(dt, x, n, c, h, w, onhip_h16_pitch(c), y, reinterpret_cast<hipStream_t>(stream));
}

int onhip_h16_to_nchw_f32(const void *x, int32_t n, int32_t c, int32_t h, int32_t w, int32_t compute, float *y, void *stream) {
    int dt, rc = h16_dtype(compute, &dt);
    if (rc) return rc;
    if (!x || !y || n < 1 || c < 1 || h < 1 || w < 1 || reinterpret_cast<uintptr_t>(x) % 16) return set_error(ONHIP_ERR_ARG, "16-bit conversion: bad argument");
    return nhwc16_to_nchw_launch(dt, x, n, c, h, w, onhip_h16_pitch(c), y, reinterpret_cast<hipStream_t>(stream));
}

int onhip_h16_from_rows_f32(const float *x, long long rows, int32_t k, int32_t compute, void *y, void *stream) {
    int dt, rc = h16_dtype(compute, &dt);
    if (rc) return rc;
    if (!x || !y || rows < 1 || k < 1) return set_error(ONHIP_ERR_ARG, "16-bit conversion: bad argument");
    return rows_to_h16_launch(dt, x, rows, k, onhip_h16_pitch(k), y, reinterpret_cast<hipStream_t>(stream));
}

int onhip_h16_to_rows_f32(const void *x, long long rows, int32_t k, int32_t compute, float *y, void *stream) {
    int dt, rc = h16_dtype(compute, &dt);
    if (rc) return rc;
    if (!x || !y || rows < 1 || k < 1) return set_error(ONHIP_ERR_ARG, "16-bit conversion: bad argument");
    return rows_from_h16_launch(dt, x, rows, k, onhip_h16_pitch(k), y, reinterpret_cast<hipStream_t>(stream));
}

// gelu != 0: lut is the GELU table and is applied whatever the descriptor says (the linear layer's fused form)
// the stored row width of the first-layer form: every output column's 8-pixel window lies inside its row
static int h16_first_width(const onhip_conv_desc_t *d, int OW) {
    const int padded = d->pad_l + d->w + d->pad_r, reach = (OW - 1) * d->stride_w + 8;
    return ((padded > reach ? padded : reach) + 1) & ~1;   // even: rows of 4-channel pixels then start on 16 bytes
}
// channels stored per pixel: 4 (8 bytes) for up to four input channels, else 8
static int h16_first_cpp(const onhip_conv_desc_t *d) { return d->cin <= 4 ? 4 : 8; }

static int h16_first_check(const onhip_conv_desc_t *d, int32_t *OH, int32_t *OW) {
    const int rc = check_conv(d, OH, OW);
    if (rc) return rc;
    if (d->group != 1 || d->cin > 8 || d->kw > 8 || d->kh > 64)
        return set_error(ONHIP_ERR_ARG, "16-bit first layer: dense, at most 8 input channels, filter rows of at most 8 columns, at most 64 of them");
    return ONHIP_OK;
}

// first != 0: x is the first-layer form [n][h][wp][cpp] and w_packed [cout][kh][8][cpp] (onhip_h16_first_*)
static int conv2d_h16_impl(const onhip_conv_desc_t *d, const void *x, const void *w_packed, const float *bias, const float *lut,
                           int gelu, const void *residual, int32_t residual_relu, void *y, int32_t y_kind, void *stream,
                           int first = 0) {
    int32_t OH, OW;
    int rc = check_conv(d, &OH, &OW);
    if (rc) return rc;
    IgemmLaunch cfg;
    memset(&cfg, 0, sizeof(cfg));
    if ((rc = h16_dtype(d->compute, &cfg.dtype))) return rc;
    if (d->group != 1) return set_error(ONHIP_ERR_ARG, "conv 16-bit: dense convolutions only");
    if (!x || !w_packed || !y || (d->has_bias && !bias)) return set_error(ONHIP_ERR_ARG, "conv 16-bit: null tensor pointer");
    if (y_kind < ONHIP_H16_OUT_NHWC || y_kind > ONHIP_H16_OUT_F32_NCHW) return set_error(ONHIP_ERR_ARG, "conv 16-bit: output kind %d", y_kind);
    if (residual && y_kind != ONHIP_H16_OUT_NHWC) return set_error(ONHIP_ERR_ARG, "conv 16-bit: the residual operand goes with the 16-bit output");
    if (residual == y) return set_error(ONHIP_ERR_ARG, "conv 16-bit: the residual operand may not be the output buffer");
    if (d->act_type == SILU && !lut) return set_error(ONHIP_ERR_ARG, "conv 16-bit: SILU needs the table");
    if (d->kh * d->kw > 64) return set_error(ONHIP_ERR_ARG, "conv 16-bit: filters of more than 64 taps are not supported");
    if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(w_packed) % 16 || reinterpret_cast<uintptr_t>(y) % 16 ||
        reinterpret_cast<uintptr_t>(residual) % 16)
        return set_error(ONHIP_ERR_ARG, "conv 16-bit: tensors must be 16-byte aligned");
    const int cp = onhip_h16_pitch(d->cin), cop = onhip_h16_pitch(d->cout);
    const int wp = first ? h16_first_width(d, OW) : d->w;
    if ((long long) d->n * d->h * wp * (first ? h16_first_cpp(d) : cp) * 2 >= (1LL << 31) || (long long) d->n * OH * OW * cop * 4 >= (1LL << 31) ||
        (long long) d->cout * d->kh * d->kw * cp * 2 >= (1LL << 31))
        return set_error(ONHIP_ERR_ARG, "conv 16-bit: tensors of 2 GiB or more are not supported");
    cfg.bl = BL_KVEC;
    cfg.batch = 1;
    IgemmParams p;
    memset(&p, 0, sizeof(p));
    p.M = d->cout;
    p.N = d->n * OH * OW;
    p.A = w_packed;
    p.B = x;
    p.H = d->h; p.OW = OW; p.OHW = OH * OW;
    p.sh = d->stride_h; p.sw = d->stride_w; p.pt = d->pad_t;
    p.use_tapmask = 1;
    if (first) {
        // A filter row is one tap of 8 pixels x 4 or 8 channels = 64 or 128 contiguous bytes of the stored row, beginning at
        // stored column ow * stride_w (the left padding is in the stored row, so no column is ever outside it); pixels are
        // 8 or 16 bytes apart.  The reduction index runs over (filter row, column, channel), zeros where the filter has none.
        p.units_per_tap = h16_first_cpp(d);
        p.tap_spans_pixels = 1;
        p.W = wp;
        p.kh = d->kh; p.kw = 1; p.khkw = d->kh;
        p.pl = 0;
        p.pix_stride = h16_first_cpp(d) * 2;
    } else {
        p.units_per_tap = cp / 8;
        p.W = d->w;
        p.kh = d->kh; p.kw = d->kw; p.khkw = d->kh * d->kw;
        p.pl = d->pad_l;
        p.pix_stride = cp * 2;
    }
    p.HW = p.H * p.W;
    p.k_units = p.khkw * p.units_per_tap;
    p.K = p.k_units * 8;
    p.lda = p.k_units * 16;      // bytes, like every quantity of the vector loader
    p.magic_kw = magic_for(p.kw); p.pass_kw = pass_for(p.kw);
    p.magic_upt = magic_for(p.units_per_tap); p.pass_upt = pass_for(p.units_per_tap);
    p.b_shift_bytes = ((long long) p.pt * p.W + p.pl) * p.pix_stride;
    p.a_slice_bytes = (long long) p.M * p.lda;
    p.b_slice_bytes = (long long) d->n * p.H * p.W * p.pix_stride;
    p.C = y;
    if (y_kind == ONHIP_H16_OUT_F32_NCHW) {
        p.out_mode = OUT_CONV;
        p.c_img_stride = (long long) d->cout * OH * OW;
        p.c_stride_m = (long long) OH * OW;
    } else {
        // element (pixel n, channel m) at n * pitch + m
        p.out_mode = OUT_PLAIN;
        p.c_stride_m = 1;
        p.c_stride_n = y_kind == ONHIP_H16_OUT_NHWC ? cop : d->cout;
        p.out_h16 = y_kind == ONHIP_H16_OUT_NHWC;
    }
    p.c_slice_bytes = (long long) d->n * OH * OW * cop * 4;
    p.bias = d->has_bias ? bias : nullptr;
    p.bias_mode = d->has_bias ? BIAS_M : BIAS_NONE;
    p.ep = make_epilogue(*d, lut);
    if (gelu) p.ep.act = ONHIP_ACT_GELU_LUT;
    p.res16 = residual;
    p.res_relu = residual_relu;
    return plan_and_launch(cfg, p, reinterpret_cast<hipStream_t>(stream));
}

int onhip_conv2d_h16(const onhip_conv_desc_t *d, const void *x, const void *w_packed, const float *bias, const float *lut,
                     const void *residual, int32_t residual_relu, void *y, int32_t y_kind, void *stream) {
    return conv2d_h16_impl(d, x, w_packed, bias, lut, 0, residual, residual_relu, y, y_kind, stream);
}

int32_t onhip_h16_first_channels(const onhip_conv_desc_t *d) { return d && onhip_h16_first_width(d) ? h16_first_cpp(d) : 0; }

int32_t onhip_h16_first_width(const onhip_conv_desc_t *d) {
    int32_t OH, OW;
    if (!d || h16_first_check(d, &OH, &OW)) return 0;
    return h16_first_width(d, OW);
}

size_t onhip_h16_first_input_bytes(const onhip_conv_desc_t *d) {
    const int32_t wp = onhip_h16_first_width(d);
    return wp ? (size_t) d->n * d->h * wp * h16_first_cpp(d) * 2 : 0;
}

size_t onhip_h16_first_weight_bytes(const onhip_conv_desc_t *d) {
    return onhip_h16_first_width(d) ? (size_t) d->cout * d->kh * 8 * h16_first_cpp(d) * 2 : 0;
}

int onhip_h16_first_from_nchw_f32(const onhip_conv_desc_t *d, const float *x, void *x_first, void *stream) {
    int32_t OH, OW;
    int dt, rc = h16_first_check(d, &OH, &OW);
    if (rc || (rc = h16_dtype(d->compute, &dt))) return rc;
    if (!x || !x_first || reinterpret_cast<uintptr_t>(x_first) % 16) return set_error(ONHIP_ERR_ARG, "16-bit first layer: null or misaligned tensor");
    return first_from_nchw_launch(dt, x, d->n, d->cin, d->h, d->w, h16_first_width(d, OW), h16_first_cpp(d), d->pad_l, x_first,
                                  reinterpret_cast<hipStream_t>(stream));
}

int onhip_h16_first_pack_weights(const onhip_conv_desc_t *d, const float *w, void *packed, void *stream) {
    int32_t OH, OW;
    int dt, rc = h16_first_check(d, &OH, &OW);
    if (rc || (rc = h16_dtype(d->compute, &dt))) return rc;
    if (!w || !packed || reinterpret_cast<uintptr_t>(packed) % 16) return set_error(ONHIP_ERR_ARG, "16-bit first layer: null or misaligned weights");
    return first_pack_w16_launch(dt, w, d->cout, d->cin, d->kh, d->kw, h16_first_cpp(d), packed, reinterpret_cast<hipStream_t>(stream));
}

int onhip_conv2d_h16_first(const onhip_conv_desc_t *d, const void *x_first, const void *w_packed, const float *bias, const float *lut,
                           void *y, int32_t y_kind, void *stream) {
    int32_t OH, OW;
    const int rc = h16_first_check(d, &OH, &OW);
    if (rc) return rc;
    return conv2d_h16_impl(d, x_first, w_packed, bias, lut, 0, nullptr, 0, y, y_kind, stream, 1);
}

int onhip_linear_h16(long long rows, int32_t k, int32_t n, int32_t compute, const void *x, const void *w_packed, const float *bias,
                     const float *gelu_lut, const void *residual, void *y, int32_t y_kind, void *stream) {
    if (rows < 1 || rows >= (1LL << 31) || k < 1 || n < 1) return set_error(ONHIP_ERR_ARG, "linear 16-bit: bad shape");
    if (y_kind == ONHIP_H16_OUT_F32_NCHW) return set_error(ONHIP_ERR_ARG, "linear 16-bit: rows come out as rows");
    // rows of a matrix are the pixels of a one-row image with k channels, the weights a 1x1 filter bank
    onhip_conv_desc_t d;
    memset(&d, 0, sizeof(d));
    d.n = 1; d.cin = k; d.h = 1; d.w = (int32_t) rows; d.cout = n; d.kh = d.kw = 1; d.stride_h = d.stride_w = 1;
    d.group = 1; d.has_bias = bias != nullptr; d.compute = compute;
    d.act_type = NOT_ACT;
    // the table GELU of device/x86/Gelu/gelu.c on the fp32 sums, as in the fp32 MatMul's fused form
    return conv2d_h16_impl(&d, x, w_packed, bias, gelu_lut, gelu_lut != nullptr, residual, 0, y, y_kind, stream);
}

// the depthwise 3x3 -> 1x1 pair at the end of a block the one-launch block kernel takes; *why (when not null) says what
// rules a pair out
static bool dw_project_shapes_ok(const onhip_conv_desc_t *dw, const onhip_conv_desc_t *pw, const char **why) {
    const char *w = nullptr;
    int32_t OH = 0, OW = 0;
    if (!dw || !pw || check_conv(dw, &OH, &OW)) w = "bad depthwise descriptor";
    else if (dw->group == 1 || dw->group != dw->cin || dw->cout != dw->cin) w = "the first convolution must be depthwise";
    else if (dw->kh != 3 || dw->kw != 3 || dw->pad_t != 1 || dw->pad_l != 1 || dw->pad_b != 1 || dw->pad_r != 1) w = "depthwise 3x3 with pads 1 only";
    else if (dw->stride_h != dw->stride_w || (dw->stride_h != 1 && dw->stride_h != 2)) w = "depthwise stride 1 or 2";
    else if (dw->cin % 16) w = "depthwise channels must be a multiple of 16";
    else if (!dw->has_bias) w = "the depthwise convolution must have a bias";
    else if (dw->compute != ONHIP_COMPUTE_F32 || pw->compute != ONHIP_COMPUTE_F32 || dw->act_type == SILU || pw->act_type == SILU) w = "fp32 without table activations";
    else if (pw->group != 1 || pw->kh != 1 || pw->kw != 1 || pw->stride_h != 1 || pw->stride_w != 1 || pw->pad_t || pw->pad_l || pw->pad_b || pw->pad_r)
        w = "the second convolution must be 1x1, stride 1, unpadded";
    else if (pw->cin != dw->cout || pw->n != dw->n || pw->h != OH || pw->w != OW) w = "the second convolution does not take the first one's output";
    else if (pw->cout < 1 || pw->cout > 128) w = "at most 128 output channels";
    else if ((long long) dw->n * dw->cin * dw->h * dw->w * 4 >= (1LL << 31) || (long long) pw->n * pw->cout * OH * OW * 4 >= (1LL << 31)) w = "tensors of 2 GiB or more";
    if (why) *why = w;
    return w == nullptr;
}

// the expansion -> depthwise -> projection triple the one-launch block kernel takes
static bool ir_block_shapes_ok(const onhip_conv_desc_t *ex, const onhip_conv_desc_t *dw, const onhip_conv_desc_t *pw, const char **why) {
    const char *w = nullptr;
    int32_t EH = 0, EW = 0, OH = 0, OW = 0;
    if (!dw_project_shapes_ok(dw, pw, &w)) {
    } else if (!ex || check_conv(ex, &EH, &EW)) w = "bad expansion descriptor";
    else if (ex->group != 1 || ex->kh != 1 || ex->kw != 1 || ex->stride_h != 1 || ex->stride_w != 1 || ex->pad_t || ex->pad_l || ex->pad_b || ex->pad_r)
        w = "the first convolution must be 1x1, stride 1, unpadded";
    else if (ex->compute != ONHIP_COMPUTE_F32 || ex->act_type == SILU || !ex->has_bias) w = "the expansion must be fp32 with a bias and no table activation";
    else if (ex->cout != dw->cin || ex->n != dw->n || ex->h != dw->h || ex->w != dw->w) w = "the depthwise convolution does not take the expansion's output";
    else if (!irblock_cin_ok(ex->cin)) w = "16, 24, 32 or 64 input channels";
    else if (pw->cout > 64) w = "at most 64 output channels";
    else if (onhip_conv_out_shape(dw, &OH, &OW) || irblock_band_rows(*dw, OH, OW, ex->cin) < 1) w = "no band of output rows fits the kernel (row length a multiple of 2, at most 128 output pixels)";
    else if ((long long) ex->n * ex->cin * ex->h * ex->w * 4 >= (1LL << 31)) w = "tensors of 2 GiB or more";
    if (why) *why = w;
    return w == nullptr;
}

int onhip_ir_block_supported(const onhip_conv_desc_t *expand, const onhip_conv_desc_t *dw, const onhip_conv_desc_t *project) {
    if (!ir_block_shapes_ok(expand, dw, project, nullptr)) return 0;
    // One workgroup per band of output rows and image, a few tens of microseconds each whatever the batch: below one
    // workgroup per compute unit the three separate launches, which spread over the whole chip, finish first (MobileNetV2
    // at batch 1: 28 workgroups).  Measured on MobileNetV2 at batch 64, one launch against three: 130 / 191 us (16 -> 96 ->
    // 24 channels, 112 x 112, stride 2), 104 / 121 (24 -> 144 -> 24, 56 x 56), 76 / 86, 44 / 54, 44 / 52.
    int32_t OH = 0, OW = 0;
    (void) onhip_conv_out_shape(dw, &OH, &OW);
    // With 64 input channels (MobileNetV2's 14 x 14 blocks, 64 -> 384 -> 64: 24 chunks of expansion per band, 256
    // workgroups at batch 64) one launch takes 65 us against 37 us for the three: taken, not recommended.
    const int rows = irblock_band_rows(*dw, OH, OW, expand->cin);
    return expand->cin <= 32 && (long long) dw->n * ((OH + rows - 1) / rows) >= 256 ? 2 : 1;
}

size_t onhip_ir_block_packed_weight_bytes(int32_t cin, int32_t ce, int32_t co) {
    return cin < 1 || ce < 1 || co < 1 ? 0 : ((size_t) ce * cin + (size_t) ce * ((co + 31) / 32 * 32)) * sizeof(float);
}

int onhip_ir_block_pack_weights(const float *expand_w, const float *project_w, int32_t cin, int32_t ce, int32_t co, float *packed, void *stream) {
    if (!expand_w || !project_w || !packed || cin < 4 || cin % 4 || ce < 16 || ce % 16 || co < 1 || reinterpret_cast<uintptr_t>(packed) % 16)
        return set_error(ONHIP_ERR_ARG, "inverted-residual block pack: bad argument");
    return irblock_pack_launch(expand_w, project_w, cin, ce, co, packed, reinterpret_cast<hipStream_t>(stream));
}

int onhip_ir_block_f32(const onhip_conv_desc_t *expand, const onhip_conv_desc_t *dw, const onhip_conv_desc_t *project, const float *x,
                       const float *packed, const float *expand_b, const float *dw_w, const float *dw_b, const float *project_b,
                       const float *residual, float *y, void *stream) {
    const char *why = nullptr;
    if (!ir_block_shapes_ok(expand, dw, project, &why)) return set_error(ONHIP_ERR_ARG, "inverted-residual block: %s", why);
    if (!x || !packed || !expand_b || !dw_w || !dw_b || !y || (project->has_bias && !project_b))
        return set_error(ONHIP_ERR_ARG, "inverted-residual block: null tensor pointer");
    if (reinterpret_cast<uintptr_t>(packed) % 16 || reinterpret_cast<uintptr_t>(x) % 16)
        return set_error(ONHIP_ERR_ARG, "inverted-residual block: input and packed weights must be 16-byte aligned");
    if (residual == y || x == y) return set_error(ONHIP_ERR_ARG, "inverted-residual block: the output buffer may not be an input");
    int32_t OH = 0, OW = 0;
    (void) onhip_conv_out_shape(dw, &OH, &OW);
    return irblock_f32_launch(*expand, *dw, *project, OH, OW, x, packed, expand_b, dw_w, dw_b, project->has_bias ? project_b : nullptr, residual,
                              make_epilogue(*expand, nullptr), make_epilogue(*dw, nullptr), make_epilogue(*project, nullptr), y,
                              reinterpret_cast<hipStream_t>(stream));
}

int onhip_attention(const onhip_attention_desc_t *d, const void *q, const void *k, const void *v, void *out, void *stream) {
    if (!d || d->batch < 1 || d->heads < 1 || d->tokens < 1) return set_error(ONHIP_ERR_ARG, "attention: bad shape");
    if (!q || !k || !v || !out) return set_error(ONHIP_ERR_ARG, "attention: null tensor pointer");
    const bool f32 = d->compute == ONHIP_COMPUTE_F32;
    int dt = DT_F32;
    if (!f32) {
        const int rc = h16_dtype(d->compute, &dt);
        if (rc) return rc;
    }
    if (d->head_dim != 64 && !(f32 && d->head_dim == 32))
        return set_error(ONHIP_ERR_ARG, "attention: head dimension %d (fp32: 32 and 64 are fused, 16-bit: 64)", d->head_dim);
    if (d->tokens > 256) return set_error(ONHIP_ERR_ARG, "attention: %d tokens (at most 256 are fused)", d->tokens);
    if ((long long) d->batch * d->heads > 65535) return set_error(ONHIP_ERR_ARG, "attention: more than 65535 (batch, head) pairs");
    const long long *strides[4] = {d->q_strides, d->k_strides, d->v_strides, d->out_strides};
    const void *ptrs[4] = {q, k, v, out};
    const int vec = f32 ? 4 : 8;   // elements of a 16-byte access
    for (int t = 0; t < 4; ++t) {
        if (reinterpret_cast<uintptr_t>(ptrs[t]) % 16) return set_error(ONHIP_ERR_ARG, "attention: tensors must be 16-byte aligned");
        for (int i = 0; i < 3; ++i)
            if (strides[t][i] < 0 || strides[t][i] % vec) return set_error(ONHIP_ERR_ARG, "attention: strides must be non-negative multiples of %d", vec);
        if (strides[t][2] < d->head_dim) return set_error(ONHIP_ERR_ARG, "attention: token stride below the head dimension");
    }
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    if (f32) return attention_f32_launch(*d, reinterpret_cast<const float *>(q), reinterpret_cast<const float *>(k),
                                         reinterpret_cast<const float *>(v), reinterpret_cast<float *>(out), st);
    return attention_h16_launch(dt, *d, q, k, v, out, st);
}

int onhip_copy_f32(const float *src, float *dst, long long n, void *stream) {
    if (!src || !dst || n < 0) return set_error(ONHIP_ERR_ARG, "copy: bad argument");
    return copy_f32_launch(src, dst, n, reinterpret_cast<hipStream_t>(stream));
}

int onhip_gemm_f32(int32_t m, int32_t k, int32_t n, const float *a, const float *w, const float *bias, float *out,
                   void *stream) {
    if (m < 1 || k < 1 || n < 1) return set_error(ONHIP_ERR_ARG, "gemm: bad shape %dx%dx%d", m, k, n);
    if (!a || !w || !bias || !out) return set_error(ONHIP_ERR_ARG, "gemm: null tensor pointer");
    // Up to eight rows of A the skinny kernel reads the weights once and is bound by that read.  More rows are a
    // matrix product worth the MFMA kernel: A [m, k] is m images of k channels and one pixel, W [n, k] the weights
    // of a 1x1 convolution, out [m, n] its NCHW result (measured at k = 2048, n = 1000: 13 us from 16 to 64 rows,
    // against 21 to 78 us).
    const long long lim = 1LL << 29;   // elements: the MFMA kernel addresses an operand with 32-bit byte offsets
    if (m > 8 && (long long) m * k < lim && (long long) m * n < lim && (long long) n * k < lim) {
        onhip_conv_desc_t d;
        memset(&d, 0, sizeof(d));
        d.n = m; d.cin = k; d.h = d.w = 1; d.cout = n; d.kh = d.kw = 1; d.stride_h = d.stride_w = 1;
        d.group = 1; d.has_bias = 1; d.act_type = NOT_ACT; d.compute = ONHIP_COMPUTE_F32;
        return conv2d_f32_impl(&d, a, w, 0, bias, nullptr, out, stream);
    }
    return gemm_nt_launch(m, k, n, a, w, bias, out, reinterpret_cast<hipStream_t>(stream));
}

}  // extern "C"
