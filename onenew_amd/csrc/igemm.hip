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
// (implicit im2col; zero padding is a predicate) or from a row-major [K, N] matrix, with lanes
// running along N so every load instruction is a coalesced run of pixels.  BL_KVEC reads 16-byte
// vectors along K from NHWC int8 activations (K ordered tap-major, channel-minor) or from an
// [N, K] matrix.  The reduction index of a load is wavefront-uniform, so its decomposition into
// (channel, tap row, tap column) costs a few multiply-high operations per wavefront, not per lane.
//
// Replaces, for the dense cases: device/x86/Conv/conv.c im2col (:168,:260) + opt_gemm.h SGEMM (:17)
// + bias sweep (:405) + do_act (:1216); the int32 GEMM and de-quantisation of conv.c:1024-1056;
// device/x86/MatMul/mat_mul.c:10.
#include "onhip_internal.hpp"

namespace onhip {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int UPT = 4;        // 16-byte units per K tile
constexpr int THREADS = 256;

template <int DT> struct Traits;
template <> struct Traits<DT_F32> {
    static constexpr int KPU = 4;
    static constexpr int RAW = 4;          // fp32 values fetched per unit
    typedef f32x16 acc_t;
    static __device__ __forceinline__ void mma(acc_t &c, const uint4 &a, const uint4 &b) {
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
    }
};
template <> struct Traits<DT_BF16> {
    static constexpr int KPU = 8;
    static constexpr int RAW = 8;
    typedef f32x16 acc_t;
    static __device__ __forceinline__ void mma(acc_t &c, const uint4 &a, const uint4 &b) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                    0, 0, 0);
    }
};
template <> struct Traits<DT_F16> {
    static constexpr int KPU = 8;
    static constexpr int RAW = 8;
    typedef f32x16 acc_t;
    static __device__ __forceinline__ void mma(acc_t &c, const uint4 &a, const uint4 &b) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                   0, 0);
    }
};
template <> struct Traits<DT_I8> {
    static constexpr int KPU = 16;
    static constexpr int RAW = 4;          // 4 dwords = 16 int8
    typedef i32x16 acc_t;
    static __device__ __forceinline__ void mma(acc_t &c, const uint4 &a, const uint4 &b) {
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

// x / d for x * d < 2^32 with magic = floor(2^32 / d) + 1; magic == 0 encodes d == 1
__device__ __forceinline__ unsigned fast_div(unsigned x, unsigned magic) {
    return magic ? __umulhi(x, magic) : x;
}

// ---- A: one unit of one row ----------------------------------------------------------------------
template <int DT>
__device__ __forceinline__ void load_a_unit(RawUnit<DT> &r, const IgemmParams &p, const char *a_base, int m, int u,
                                            bool in_range) {
    constexpr int KPU = Traits<DT>::KPU;
    if constexpr (DT == DT_I8) {
        // packed weights: every row holds k_units whole units, zero padded
        r.q = make_uint4(0, 0, 0, 0);
        if (in_range && m < p.M) r.q = *reinterpret_cast<const uint4 *>(a_base + ((size_t) m * p.lda + (size_t) u * 16));
    } else {
        const float *row = reinterpret_cast<const float *>(a_base) + (size_t) m * p.lda;
        const int k = u * KPU;
        const bool row_ok = in_range && m < p.M;
        if (p.a_vec) {
#pragma unroll
            for (int q = 0; q < KPU / 4; ++q) {
                f32x4 t = {0.f, 0.f, 0.f, 0.f};
                if (row_ok && k + 4 * q < p.K) t = *reinterpret_cast<const f32x4 *>(row + k + 4 * q);
                r.v[4 * q] = t.x; r.v[4 * q + 1] = t.y; r.v[4 * q + 2] = t.z; r.v[4 * q + 3] = t.w;
            }
        } else {
#pragma unroll
            for (int e = 0; e < KPU; ++e) r.v[e] = (row_ok && k + e < p.K) ? row[k + e] : 0.0f;
        }
    }
}

// ---- B: per-thread column state, fixed for the whole K loop -------------------------------------
struct ColState {
    int base;      // element (gather) or byte (kvec) offset of the column's origin; may be negative
    int ih0, iw0;  // top-left input coordinate of the receptive field
    bool valid;
};

template <int BL>
__device__ __forceinline__ ColState make_col(const IgemmParams &p, int n) {
    ColState c;
    c.valid = n < p.N;
    const int nn = c.valid ? n : 0;
    const int img = nn / p.OHW;
    const int pix = nn - img * p.OHW;
    const int oh = pix / p.OW;
    const int ow = pix - oh * p.OW;
    c.ih0 = oh * p.sh - p.pt;
    c.iw0 = ow * p.sw - p.pl;
    if constexpr (BL == BL_GATHER) {
        c.base = img * (int) p.b_img_stride + c.ih0 * p.W + c.iw0;
    } else {
        c.base = ((img * p.H + c.ih0) * p.W + c.iw0) * p.pix_stride;
    }
    return c;
}

template <int DT, int BL>
__device__ __forceinline__ void load_b_unit(RawUnit<DT> &r, const IgemmParams &p, const char *b_base,
                                            const ColState &c, int u, bool in_range) {
    constexpr int KPU = Traits<DT>::KPU;
    if constexpr (BL == BL_GATHER) {
        static_assert(DT != DT_I8, "int8 activations are staged as NHWC vectors");
        const float *x = reinterpret_cast<const float *>(b_base);
#pragma unroll
        for (int e = 0; e < KPU; ++e) {
            const unsigned k = (unsigned) (u * KPU + e);  // wavefront-uniform
            int off, ih, iw;
            if (p.khkw == 1) {
                off = (int) k * p.HW;
                ih = c.ih0;
                iw = c.iw0;
            } else {
                const unsigned ch = fast_div(k, p.magic_khkw);
                const unsigned rem = k - ch * (unsigned) p.khkw;
                const unsigned i = fast_div(rem, p.magic_kw);
                const unsigned j = rem - i * (unsigned) p.kw;
                off = (int) ch * p.HW + (int) i * p.W + (int) j;
                ih = c.ih0 + (int) i;
                iw = c.iw0 + (int) j;
            }
            const bool ok = in_range && c.valid && (int) k < p.K && (unsigned) ih < (unsigned) p.H &&
                            (unsigned) iw < (unsigned) p.W;
            r.v[e] = ok ? x[c.base + off] : 0.0f;
        }
    } else {
        // unit -> (tap, channel block); tap -> (i, j)
        int off, ih, iw;
        bool tap_ok = true;
        if (p.khkw == 1) {
            off = u * 16;
            ih = c.ih0;
            iw = c.iw0;
        } else {
            const unsigned tap = fast_div((unsigned) u, p.magic_upt);
            const unsigned cb = (unsigned) u - tap * (unsigned) p.units_per_tap;
            const unsigned i = fast_div(tap, p.magic_kw);
            const unsigned j = tap - i * (unsigned) p.kw;
            tap_ok = (int) tap < p.khkw;
            off = ((int) i * p.W + (int) j) * p.pix_stride + (int) cb * 16;
            ih = c.ih0 + (int) i;
            iw = c.iw0 + (int) j;
        }
        const bool ok = in_range && tap_ok && c.valid && (unsigned) ih < (unsigned) p.H && (unsigned) iw < (unsigned) p.W;
        uint4 q = make_uint4(0, 0, 0, 0);
        if (ok) q = *reinterpret_cast<const uint4 *>(b_base + c.base + off);
        if constexpr (DT == DT_I8) {
            r.q = q;
        } else {
            static_assert(DT == DT_F32 || DT == DT_I8, "vector B loader carries raw 16-byte units");
            r.v[0] = __uint_as_float(q.x); r.v[1] = __uint_as_float(q.y);
            r.v[2] = __uint_as_float(q.z); r.v[3] = __uint_as_float(q.w);
        }
    }
}

// ---- epilogue of one element ----------------------------------------------------------------------
__device__ __forceinline__ long long out_offset(const IgemmParams &p, int batch, int m, int n) {
    if (p.out_mode == OUT_CONV) {
        const int img = n / p.OHW;
        const int pix = n - img * p.OHW;
        return (long long) batch * p.c_batch_stride + (long long) img * p.c_img_stride + (long long) m * p.c_stride_m + pix;
    }
    return (long long) batch * p.c_batch_stride + (long long) m * p.c_stride_m + (long long) n * p.c_stride_n;
}

// fp32 accumulators: bias after the full sum, then activation (conv.c:405-412, :61-63)
__device__ __forceinline__ void finish_f32(const IgemmParams &p, long long off, int m, int n, float v) {
    if (p.bias_mode == BIAS_M) v = __fadd_rn(v, p.bias[m]);
    else if (p.bias_mode == BIAS_N) v = __fadd_rn(v, p.bias[n]);
    v = apply_act(v, p.ep);
    reinterpret_cast<float *>(p.C)[off] = v;
}

// int32 accumulators: conv.c:1041-1056, three separately rounded fp32 operations, then the
// activation and, optionally, the consumer's quantisation (conv.c:961-973)
__device__ __forceinline__ void finish_i32(const IgemmParams &p, long long off, int m, int acc) {
    if (p.acc_out) p.acc_out[off] = acc;
    float f = __fmul_rn((float) acc, p.in_scale);
    if (p.bias32) f = __fadd_rn(f, (float) p.bias32[m]);
    const float coeff = __fdiv_rn(p.weight_aux[m], 127.0f);
    float y = apply_act(__fmul_rn(f, coeff), p.ep);
    if (p.out_s8) {
        float t = __fmul_rn(y, p.out_inv_scale);
        t = (t < -128.0f) ? -128.0f : (t > 127.0f) ? 127.0f : t;
        reinterpret_cast<int8_t *>(p.C)[off] = (int8_t) roundf(t);
    } else {
        reinterpret_cast<float *>(p.C)[off] = y;
    }
}

// ---- the kernel --------------------------------------------------------------------------------
template <int DT, int BL, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(THREADS) void igemm_kernel(const IgemmParams p) {
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    static_assert(TM >= 1 && TN >= 1 && BM % (WM * 32) == 0 && BN % (WN * 32) == 0, "tile / wave grid mismatch");
    static_assert(THREADS % BN == 0 || BN % THREADS == 0, "B loader mapping");
    constexpr int A_SLOTS = BM * UPT, B_SLOTS = BN * UPT;
    constexpr int A_PER_T = (A_SLOTS + THREADS - 1) / THREADS;
    constexpr int B_PER_T = B_SLOTS / THREADS;
    static_assert(B_PER_T >= 1, "BN >= 64");
    typedef typename Traits<DT>::acc_t acc_t;

    __shared__ uint4 lds[2][A_SLOTS + B_SLOTS];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lh = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    // XCD-aware tile order: consecutive workgroup ids go round-robin over the 8 XCDs (each with its
    // own L2); give every XCD a contiguous run of tiles so neighbours in (m, n) share an L2.
    const int tiles_m = (p.M + BM - 1) / BM;
    int lid;
    {
        const int nb = gridDim.x, bid = blockIdx.x;
        const int q = nb >> 3, rmd = nb & 7, xcd = bid & 7, idx = bid >> 3;
        lid = xcd * q + (xcd < rmd ? xcd : rmd) + idx;
    }
    const int tile_m = lid % tiles_m, tile_n = lid / tiles_m;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int batch = blockIdx.z;
    const int u_begin = blockIdx.y * p.k_split_units;
    const int u_end = min(p.k_units, u_begin + p.k_split_units);
    const int k_tiles = (u_end - u_begin + UPT - 1) / UPT;

    const char *a_base = reinterpret_cast<const char *>(p.A) +
                         (size_t) batch * p.a_batch_stride * (DT == DT_I8 ? 1 : 4);
    const char *b_base = reinterpret_cast<const char *>(p.B) +
                         (size_t) batch * p.b_batch_stride * ((DT == DT_I8) ? 1 : 4);

    // B column of this thread (same for all of its units)
    const ColState col = make_col<BL>(p, n0 + (tid % BN));

    acc_t acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;

    RawUnit<DT> ra[A_PER_T], rb[B_PER_T];

    auto fetch = [&](int kt) {
        const int ub = u_begin + kt * UPT;
#pragma unroll
        for (int t = 0; t < A_PER_T; ++t) {
            const int f = tid + t * THREADS;
            const int ml = f / UPT, ua = f % UPT;
            const bool slot_ok = (A_SLOTS % THREADS == 0) || f < A_SLOTS;
            load_a_unit<DT>(ra[t], p, a_base, m0 + ml, ub + ua, slot_ok && ub + ua < u_end);
        }
#pragma unroll
        for (int t = 0; t < B_PER_T; ++t) {
            const int uu = __builtin_amdgcn_readfirstlane((tid + t * THREADS) / BN);
            load_b_unit<DT, BL>(rb[t], p, b_base, col, ub + uu, ub + uu < u_end);
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int t = 0; t < A_PER_T; ++t) {
            const int f = tid + t * THREADS;
            const int ml = f / UPT, ua = f % UPT;
            if ((A_SLOTS % THREADS == 0) || f < A_SLOTS) lds[buf][ua * BM + ml] = pack_unit<DT>(ra[t]);
        }
#pragma unroll
        for (int t = 0; t < B_PER_T; ++t) {
            const int f = tid + t * THREADS;
            lds[buf][A_SLOTS + (f / BN) * BN + (f % BN)] = pack_unit<DT>(rb[t]);
        }
    };

    if (k_tiles > 0) {
        fetch(0);
        stage(0);
    }
    __syncthreads();

    for (int kt = 0; kt < k_tiles; ++kt) {
        const int buf = kt & 1;
        const bool more = kt + 1 < k_tiles;
        if (more) fetch(kt + 1);
#pragma unroll
        for (int s = 0; s < UPT / 2; ++s) {
            uint4 av[TM], bv[TN];
#pragma unroll
            for (int a = 0; a < TM; ++a) av[a] = lds[buf][(2 * s + lh) * BM + wm * (BM / WM) + a * 32 + li];
#pragma unroll
            for (int b = 0; b < TN; ++b) bv[b] = lds[buf][A_SLOTS + (2 * s + lh) * BN + wn * (BN / WN) + b * 32 + li];
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int b = 0; b < TN; ++b) Traits<DT>::mma(acc[a][b], av[a], bv[b]);
        }
        if (more) stage(buf ^ 1);
        __syncthreads();
    }

    // epilogue: lane (li, lh) of a 32x32 block holds column li and rows 8*(r/4) + 4*lh + (r%4)
#pragma unroll
    for (int b = 0; b < TN; ++b) {
        const int n = n0 + wn * (BN / WN) + b * 32 + li;
        if (n >= p.N) continue;
        const long long col_off = out_offset(p, batch, 0, n);
#pragma unroll
        for (int a = 0; a < TM; ++a) {
            const int mb = m0 + wm * (BM / WM) + a * 32 + 4 * lh;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = mb + 8 * (r / 4) + (r % 4);
                if (m >= p.M) continue;
                const long long off = col_off + (long long) m * p.c_stride_m;
                if (p.partial) {
                    // split-K: raw partial sums [split][batch][M][N]; the reduce kernel finishes
                    const size_t po = (((size_t) blockIdx.y * gridDim.z + batch) * p.M + m) * (size_t) p.N + n;
                    if constexpr (DT == DT_I8) reinterpret_cast<int *>(p.partial)[po] = acc[a][b][r];
                    else p.partial[po] = acc[a][b][r];
                } else if constexpr (DT == DT_I8) {
                    finish_i32(p, off, m, acc[a][b][r]);
                } else {
                    finish_f32(p, off, m, n, acc[a][b][r]);
                }
            }
        }
    }
}

// sums the split-K partials in split order and applies the epilogue
template <bool IS_INT>
__global__ __launch_bounds__(256) void splitk_finish_kernel(const IgemmParams p, int split, int batches) {
    const long long total = (long long) batches * p.M * p.N;
    const long long idx = (long long) blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int n = (int) (idx % p.N);
    const long long t = idx / p.N;
    const int m = (int) (t % p.M);
    const int batch = (int) (t / p.M);
    const long long off = out_offset(p, batch, m, n);
    if constexpr (IS_INT) {
        int acc = 0;
        for (int s = 0; s < split; ++s) acc += reinterpret_cast<const int *>(p.partial)[(size_t) s * total + idx];
        finish_i32(p, off, m, acc);
    } else {
        float acc = 0.0f;
        for (int s = 0; s < split; ++s) acc = __fadd_rn(acc, p.partial[(size_t) s * total + idx]);
        finish_f32(p, off, m, n, acc);
    }
}

// ---- host side -----------------------------------------------------------------------------------
template <int DT, int BL, int BM, int BN, int WM, int WN>
static int launch_one(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    const int tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
    dim3 grid(tiles, cfg.split, cfg.batch);
    hipLaunchKernelGGL((igemm_kernel<DT, BL, BM, BN, WM, WN>), grid, dim3(THREADS), 0, stream, p);
    ONHIP_CHECK_HIP(hipGetLastError());
    if (p.partial) {
        IgemmParams q = p;
        const long long total = (long long) cfg.batch * p.M * p.N;
        const int blocks = (int) ((total + 255) / 256);
        if (DT == DT_I8)
            hipLaunchKernelGGL((splitk_finish_kernel<true>), dim3(blocks), dim3(256), 0, stream, q, cfg.split, cfg.batch);
        else
            hipLaunchKernelGGL((splitk_finish_kernel<false>), dim3(blocks), dim3(256), 0, stream, q, cfg.split, cfg.batch);
        ONHIP_CHECK_HIP(hipGetLastError());
    }
    return ONHIP_OK;
}

template <int DT, int BL>
static int launch_tile(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    const int key = cfg.bm * 1000 + cfg.bn;
    switch (key) {
        case 128128: return launch_one<DT, BL, 128, 128, 2, 2>(cfg, p, stream);
        case 64128: return launch_one<DT, BL, 64, 128, 2, 2>(cfg, p, stream);
        case 128064: return launch_one<DT, BL, 128, 64, 2, 2>(cfg, p, stream);
        case 64064: return launch_one<DT, BL, 64, 64, 2, 2>(cfg, p, stream);
        case 32128: return launch_one<DT, BL, 32, 128, 1, 4>(cfg, p, stream);
        case 32256: return launch_one<DT, BL, 32, 256, 1, 4>(cfg, p, stream);
        default: return set_error(ONHIP_ERR_ARG, "igemm: no kernel for tile %dx%d", cfg.bm, cfg.bn);
    }
}

int igemm_launch(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    if (p.M < 1 || p.N < 1 || p.k_units < 1 || cfg.batch < 1 || cfg.split < 1)
        return set_error(ONHIP_ERR_ARG, "igemm: empty problem M=%d N=%d units=%d", p.M, p.N, p.k_units);
    if (cfg.batch > 65535 || cfg.split > 65535) return set_error(ONHIP_ERR_ARG, "igemm: grid too large");
    if (cfg.split > 1 && !p.partial) return set_error(ONHIP_ERR_WORKSPACE, "igemm: split-K without workspace");
    switch (cfg.dtype * 2 + cfg.bl) {
        case DT_F32 * 2 + BL_GATHER: return launch_tile<DT_F32, BL_GATHER>(cfg, p, stream);
        case DT_F32 * 2 + BL_KVEC: return launch_tile<DT_F32, BL_KVEC>(cfg, p, stream);
        case DT_BF16 * 2 + BL_GATHER: return launch_tile<DT_BF16, BL_GATHER>(cfg, p, stream);
        case DT_F16 * 2 + BL_GATHER: return launch_tile<DT_F16, BL_GATHER>(cfg, p, stream);
        case DT_I8 * 2 + BL_KVEC: return launch_tile<DT_I8, BL_KVEC>(cfg, p, stream);
        default: return set_error(ONHIP_ERR_ARG, "igemm: unsupported dtype %d / loader %d", cfg.dtype, cfg.bl);
    }
}

// Tile choice: largest tile whose padding waste is small and that still yields enough workgroups to
// cover the 256 CUs a few times over.
void igemm_pick_tile(IgemmLaunch &cfg, const IgemmParams &p) {
    static const int cand[][2] = {{128, 128}, {64, 128}, {128, 64}, {64, 64}, {32, 128}, {32, 256}};
    static const double weight[] = {1.0, 0.9, 0.88, 0.75, 0.7, 0.8};
    double best = -1.0;
    for (int i = 0; i < 6; ++i) {
        const int bm = cand[i][0], bn = cand[i][1];
        const long long tm = (p.M + bm - 1) / bm, tn = (p.N + bn - 1) / bn;
        const double eff = ((double) p.M * p.N) / ((double) tm * bm * tn * bn);
        const double wgs = (double) tm * tn * cfg.batch;
        const double fill = wgs >= 512.0 ? 1.0 : (wgs / 512.0);
        const double score = eff * weight[i] * (0.25 + 0.75 * fill);
        if (score > best) { best = score; cfg.bm = bm; cfg.bn = bn; }
    }
    cfg.split = 1;
}

}  // namespace onhip
