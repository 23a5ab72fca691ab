// fp32 GEMM kernel for the plain loader's problems (1x1 stride-1 unpadded convolutions, row-major matrix
// products) whose B rows are contiguous along N: B never passes through LDS.
//
// The tiled kernel (igemm_kernel.hpp) spends its steady state on LDS traffic: per 8 MFMAs a wavefront issues 2 LDS
// stores and 4 LDS reads of 16 bytes per lane, and a model loop with exactly that mix reaches about 70 % of the MFMA
// rate where the MFMAs alone reach 97 %.  Here a lane loads 16 bytes = four neighbouring columns of one row of B
// straight from global memory and uses them as the B operand of four MFMAs: block j of a wavefront covers the columns
// {4 * lane + j}, so the wavefront's tile is 32 rows x 128 columns in four column-interleaved 32x32 blocks.  An MFMA
// step takes k = p and k = p + 4 of an 8-deep slab for its two lane halves, which makes a lane's four A values
// 16 contiguous bytes; A (small) still goes through LDS, one 16-byte read per 16 MFMAs.  Per 32 MFMAs a wavefront
// issues 8 global B loads, 2 LDS reads and the workgroup's share of A: an eighth of the tiled kernel's LDS
// instructions per MFMA.  The result of a lane is four neighbouring columns per row: 16-byte stores.
//
// Conditions (rowb_f32_ok): fp32, plain loader with unit strides, K, N and the pixels per image multiples of 4
// (column quads never straddle an image or a row of B, A units are whole), unit column stride of C.  K is split only
// for the tiles left over after whole rounds of 256 (dp_tiles / tail_tiles as in igemm_kernel).
#include "igemm_kernel.hpp"

namespace onhip {

// K tile: 16 reduction steps = 2 slabs of 8; A units per row and tile: 4
constexpr int RB_KT = 16;

// sbias: the per-row bias of this wavefront's 32 rows in LDS (-0.0f, the addend that changes nothing, without one)
template <int EPI>
__device__ __forceinline__ void rowb_store(const IgemmParams &p, f32x16 (&acc)[4], int batch, int m_wave, int n_quad, int lh,
                                           const float *sbias) {
    const rsrc_t rc = make_rsrc(reinterpret_cast<const char *>(p.C) + (size_t) batch * p.c_batch_stride * 4, RSRC_RANGE);
    const bool col_ok = n_quad < p.N;
    const int nn = col_ok ? n_quad : 0;
    const unsigned col_voff = col_ok ? out_col_offset(p, nn, 4) + (unsigned) (4 * lh) * (unsigned) p.c_stride_m * 4u : OOB;
    const bool bias_n_on = p.bias_mode == BIAS_N;
    const rsrc_t rbias_n = make_rsrc(p.bias, bias_n_on ? (unsigned) (p.N * 4) : 0u);
    const uint4 bn = buf_load_b128(rbias_n, (unsigned) nn * 4u, 0);
    const float bias_n[4] = {__uint_as_float(bn.x), __uint_as_float(bn.y), __uint_as_float(bn.z), __uint_as_float(bn.w)};
    const bool m_edge = m_wave + 32 > p.M;
    float bias_m[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float4 t = *reinterpret_cast<const float4 *>(sbias + 8 * q + 4 * lh);
        bias_m[4 * q + 0] = t.x; bias_m[4 * q + 1] = t.y; bias_m[4 * q + 2] = t.z; bias_m[4 * q + 3] = t.w;
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int m_uni = m_wave + 8 * (r / 4) + (r % 4);   // row of the lanes with lh == 0
        const bool row_ok = !m_edge || m_uni + 4 * lh < p.M;
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // one add whatever the bias: the row's (or -0.0f) unless the launch has a per-column one
            v[j] = act_fast<EPI>(__fadd_rn(acc[j][r], bias_n_on ? bias_n[j] : bias_m[r]), p.ep);
        }
        // row offset in the vector offset, scalar offset the constant 0: a 128-bit buffer store with a register as its
        // scalar offset gets no gap from the compiler before the next write to its data registers, which on this GPU can
        // change what some lanes store
        __builtin_amdgcn_raw_buffer_store_b128(u32x4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]),
                                                     __float_as_uint(v[3])},
                                               rc, row_ok ? col_voff + (unsigned) m_uni * (unsigned) p.c_stride_m * 4u : OOB, 0, 0);
    }
}

// raw sums of one K slice: [slice][M][N - part_begin], four columns per store
__device__ __forceinline__ void rowb_store_partial(const IgemmParams &p, f32x16 (&acc)[4], int slice, int m_wave, int n_quad, int lh) {
    const int width = p.N - p.part_begin;
    const rsrc_t rp = make_rsrc(reinterpret_cast<const char *>(p.partial) + (size_t) slice * p.M * width * 4, RSRC_RANGE);
    const unsigned cv = n_quad < p.N ? (unsigned) (n_quad - p.part_begin + 4 * lh * width) * 4u : OOB;
    const bool m_edge = m_wave + 32 > p.M;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int m_uni = m_wave + 8 * (r / 4) + (r % 4);
        const bool row_ok = !m_edge || m_uni + 4 * lh < p.M;
        const float v0 = acc[0][r], v1 = acc[1][r], v2 = acc[2][r], v3 = acc[3][r];
        __builtin_amdgcn_raw_buffer_store_b128(u32x4{__float_as_uint(v0), __float_as_uint(v1), __float_as_uint(v2), __float_as_uint(v3)},
                                               rp, row_ok ? cv + (unsigned) m_uni * (unsigned) width * 4u : OOB, 0, 0);
    }
}

template <int WM, int WN>
__global__ __launch_bounds__(64 * WM * WN) void rowb_f32_kernel(const IgemmParams p) {
    constexpr int NT = 64 * WM * WN, BM = 32 * WM, BN = 128 * WN;
    constexpr int A_SLOTS = BM * 4, A_PER_T = (A_SLOTS + NT - 1) / NT;
    constexpr int A_LD = BM + 1;   // a spare slot per unit row: the four units of a row are stored by neighbouring threads
    __shared__ uint4 lds[2][4 * A_LD];
    __shared__ __attribute__((aligned(16))) float s_bias[BM];   // the tile's rows of a per-row bias, for the store

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;
    const int tiles_m = (p.M + BM - 1) / BM;
    // workgroup -> (tile, K slice): whole tiles first, then the slices of the leftover tiles (see igemm_kernel)
    int lid, slice = 0;
    bool whole_k = true;
    {
        const int bid = blockIdx.x;
        if (p.dp_tiles > 0 && bid >= p.dp_tiles) {
            const int r = bid - p.dp_tiles;
            slice = r / p.tail_tiles;
            lid = p.dp_tiles + (r - slice * p.tail_tiles);
            whole_k = false;
        } else {   // every XCD gets a contiguous run of tiles (its own L2)
            const int nb = p.dp_tiles > 0 ? p.dp_tiles : (int) gridDim.x;
            const int q = nb >> 3, rmd = nb & 7, xcd = bid & 7, idx = bid >> 3;
            lid = xcd * q + (xcd < rmd ? xcd : rmd) + idx;
        }
    }
    const int tile_n = (int) div31((unsigned) lid, p.div_tiles_m), tile_m = lid - tile_n * tiles_m;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int batch = blockIdx.z;
    // the slice's K tiles; a slice is a whole number of K tiles (4 units of 16 bytes each)
    const int kt_begin = whole_k ? 0 : slice * p.k_split_units / 4;
    const int k_end = whole_k ? p.K : min(p.K, (slice + 1) * p.k_split_units * 4);
    const int k_tiles = (k_end + RB_KT - 1) / RB_KT - kt_begin;   // tiles of this workgroup, numbered from 0

    const char *a_base = reinterpret_cast<const char *>(p.A) + (size_t) batch * p.a_batch_stride * 4;
    const char *b_base = reinterpret_cast<const char *>(p.B) + (size_t) batch * p.b_batch_stride * 4;
    const unsigned a_bytes = (unsigned) p.a_slice_bytes, b_bytes = (unsigned) p.b_slice_bytes;

    // A: (row, unit) slots of the workgroup's tile
    unsigned a_voff[A_PER_T];
    int a_unit[A_PER_T];
#pragma unroll
    for (int t = 0; t < A_PER_T; ++t) {
        const int f = tid + t * NT, ml = f / 4, ua = f % 4;
        const bool ok = ((A_SLOTS % NT == 0) || f < A_SLOTS) && m0 + ml < p.M;
        a_unit[t] = ua;
        a_voff[t] = ok ? (unsigned) ((m0 + ml) * p.lda + ua * 4) * 4u : OOB;
    }
    // B: this lane's four columns; its half of the wavefront reads rows k + 4 * lh of every 8-deep slab
    const int n_quad = n0 + wn * 128 + 4 * li;
    unsigned b_voff;
    {
        const bool ok = n_quad < p.N;
        const int nn = ok ? n_quad : 0;
        const int img = (int) div31((unsigned) nn, p.div_ohw), pix = nn - img * p.OHW;
        b_voff = ok ? (unsigned) (img * (int) p.b_img_stride + pix + 4 * lh * p.HW) * 4u : OOB;
    }
    const unsigned row_bytes = (unsigned) p.HW * 4u;

    f32x16 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;

    uint4 qa[A_PER_T];          // A units on their way to LDS
    uint4 qb0[8], qb1[8];       // B rows of two K tiles: [slab * 4 + step]
    uint4 oa0[2], oa1[2];       // A operands of two K tiles: one unit per slab

    auto issue_a = [&](int kt) __attribute__((always_inline)) {
        const rsrc_t ra = make_rsrc(a_base, kt < k_tiles ? a_bytes : 0u);
        const int k0 = (kt_begin + kt) * RB_KT;
#pragma unroll
        for (int t = 0; t < A_PER_T; ++t)   // K and the slices are multiples of 4: a unit lies inside or outside as a whole
            qa[t] = buf_load_b128(ra, (k0 + a_unit[t] * 4) < k_end ? a_voff[t] : OOB, (unsigned) (k0 * 4));
    };
    auto stage_a = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < A_PER_T; ++t) {
            const int f = tid + t * NT;
            if ((A_SLOTS % NT == 0) || f < A_SLOTS) lds[buf][(f % 4) * A_LD + f / 4] = qa[t];
        }
    };
    // rows past the end of K or of the slice are read like any other (they hold finite tensor data or lie outside the
    // buffer and read as zero); A is zero there.  A tile past the end is switched off as a whole.
    auto issue_b = [&](uint4 (&qb)[8], int kt, int slab) __attribute__((always_inline)) {
        const rsrc_t rb = make_rsrc(b_base, kt < k_tiles ? b_bytes : 0u);
#pragma unroll
        for (int s = 0; s < 4; ++s)
            qb[slab * 4 + s] = buf_load_b128(rb, b_voff, (unsigned) ((kt_begin + kt) * RB_KT + slab * 8 + s) * row_bytes);
    };
    auto read_a = [&](uint4 (&oa)[2], int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int slab = 0; slab < 2; ++slab) oa[slab] = lds[buf][(2 * slab + lh) * A_LD + wm * 32 + li];
    };
    auto comp = [](const uint4 &q, int i) __attribute__((always_inline)) {
        return __uint_as_float(i == 0 ? q.x : i == 1 ? q.y : i == 2 ? q.z : q.w);
    };
    // one K tile: 32 MFMAs.  In their shadow: LDS store of A of tile kt+1, global loads of A of tile kt+2 and, slab
    // by slab as the registers come free, of B of tile kt+2; barrier at mid-tile, then the A operands of tile kt+1.
    auto body = [&](uint4 (&qb)[8], uint4 (&oa)[2], uint4 (&oa_next)[2], int kt) __attribute__((always_inline)) {
        const int nbuf = (kt + 1) & 1;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int slab = 0; slab < 2; ++slab) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(comp(oa[slab], s), comp(qb[slab * 4 + s], j), acc[j], 0, 0, 0);
                if (slab == 0 && s == 0) {
                    stage_a(nbuf);
                    issue_a(kt + 2);
                }
            }
            issue_b(qb, kt + 2, slab);
            if (slab == 0) __syncthreads();
            else read_a(oa_next, nbuf);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    issue_a(0);
    issue_b(qb0, 0, 0);
    issue_b(qb0, 0, 1);
    stage_a(0);
    issue_a(1);
    issue_b(qb1, 1, 0);
    issue_b(qb1, 1, 1);
    // the bias rows behind the first operand loads; in LDS when the K loop is over
    float bias_row;
    {
        const bool on = p.bias_mode == BIAS_M;
        const float bv = buf_load_f32(make_rsrc(p.bias, on ? (unsigned) (p.M * 4) : 0u), tid < BM ? (unsigned) (m0 + tid) * 4u : OOB, 0);
        bias_row = on ? bv : -0.0f;
    }
    __syncthreads();
    read_a(oa0, 0);
    int kt = 0;
    for (; kt + 2 <= k_tiles; kt += 2) {
        body(qb0, oa0, oa1, kt);
        body(qb1, oa1, oa0, kt + 1);
    }
    if (kt < k_tiles) body(qb0, oa0, oa1, kt);

    const int m_wave = m0 + wm * 32;
    if (!whole_k) {
        rowb_store_partial(p, acc, slice, m_wave, n_quad, lh);
        return;
    }
    if (tid < BM) s_bias[tid] = bias_row;
    __syncthreads();
    const float *sbias = s_bias + wm * 32;
    switch (p.ep.act) {
        case NOT_ACT:
        case RELU6: rowb_store<EPI_NONE>(p, acc, batch, m_wave, n_quad, lh, sbias); break;
        case RELU: rowb_store<EPI_RELU>(p, acc, batch, m_wave, n_quad, lh, sbias); break;
        case CLIP: rowb_store<EPI_CLIP>(p, acc, batch, m_wave, n_quad, lh, sbias); break;
        case SILU:
        case ONHIP_ACT_GELU_LUT: rowb_store<EPI_LUT>(p, acc, batch, m_wave, n_quad, lh, sbias); break;
        default: rowb_store<EPI_GENERIC>(p, acc, batch, m_wave, n_quad, lh, sbias); break;
    }
}

bool rowb_f32_ok(const IgemmLaunch &cfg, const IgemmParams &p) {
    if (cfg.dtype != DT_F32 || cfg.bl != BL_PLAIN) return false;
    if (p.sh != 1 || p.sw != 1 || p.OHW != p.HW) return false;
    if ((p.K % 4) || (p.N % 4) || (p.OHW % 4) || (p.HW % 4)) return false;
    if (p.out_mode == OUT_PLAIN && p.c_stride_n != 1) return false;
    if (p.lda % 4) return false;
    if (p.res) return false;   // the store has no registers to spare for a residual operand: the tiled kernel takes those
    return true;
}

template <int WM, int WN>
static int rowb_launch_one(const IgemmLaunch &cfg, const IgemmParams &p_in, hipStream_t stream) {
    constexpr int BM = 32 * WM, BN = 128 * WN;
    IgemmParams p = p_in;
    const int tiles_m = (p.M + BM - 1) / BM;
    const long long tiles = (long long) tiles_m * ((p.N + BN - 1) / BN);
    if (tiles > 0x7fffffffLL) return set_error(ONHIP_ERR_ARG, "igemm: grid too large");
    p.div_ohw = make_div31((unsigned) (p.OHW > 0 ? p.OHW : 1));
    p.div_ow = make_div31((unsigned) (p.OW > 0 ? p.OW : 1));
    p.div_tiles_m = make_div31((unsigned) tiles_m);
    unsigned grid_x = (unsigned) tiles;
    if (p.dp_tiles > 0) {   // whole tiles, then cfg.split K slices of each leftover tile
        if (cfg.batch != 1 || p.dp_tiles + p.tail_tiles != tiles || !p.partial || cfg.split < 2 || (p.k_split_units % 4) ||
            p.part_begin != p.dp_tiles / tiles_m * BN || p.M > 4 * 65535)
            return set_error(ONHIP_ERR_ARG, "igemm: inconsistent leftover-tile launch");
        grid_x = (unsigned) (p.dp_tiles + p.tail_tiles * cfg.split);
    }
    hipLaunchKernelGGL((rowb_f32_kernel<WM, WN>), dim3(grid_x, 1, cfg.batch), dim3(64 * WM * WN), 0, stream, p);
    ONHIP_CHECK_HIP(hipGetLastError());
    if (p.dp_tiles > 0) {
        const dim3 fgrid((p.N - p.part_begin + 63) / 64, (p.M + 3) / 4, 1);
        hipLaunchKernelGGL((splitk_finish_kernel<false>), fgrid, dim3(64, 4), 0, stream, p, cfg.split, 1);
        ONHIP_CHECK_HIP(hipGetLastError());
    }
    return ONHIP_OK;
}

// cfg.bm x cfg.bn names the workgroup tile: 64x128 (2 wavefronts), 128x128 (4, stacked along M), 64x256 (2 x 2),
// 96x128 (3 stacked), 32x256 and 32x512 (2 and 4 side by side)
int rowb_f32_launch(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    if (!rowb_f32_ok(cfg, p) || (p.dp_tiles > 0) != (cfg.split > 1) || (p.dp_tiles > 0) != (p.partial != nullptr))
        return set_error(ONHIP_ERR_ARG, "igemm: the row-B kernel does not take this problem");
    if (p.a_slice_bytes >= (1LL << 31) || p.b_slice_bytes >= (1LL << 31) || p.c_slice_bytes >= (1LL << 31))
        return set_error(ONHIP_ERR_ARG, "igemm: an operand slice of 2 GiB or more is not supported");
    switch (cfg.bm * 1000 + cfg.bn) {
        case 64128: return rowb_launch_one<2, 1>(cfg, p, stream);
        case 128128: return rowb_launch_one<4, 1>(cfg, p, stream);
        case 64256: return rowb_launch_one<2, 2>(cfg, p, stream);
        case 96128: return rowb_launch_one<3, 1>(cfg, p, stream);   // six-fold channel expansions are multiples of 96
        case 32256: return rowb_launch_one<1, 2>(cfg, p, stream);   // few output channels (projection layers)
        case 32512: return rowb_launch_one<1, 4>(cfg, p, stream);
        default: return set_error(ONHIP_ERR_ARG, "igemm: no row-B kernel for tile %dx%d", cfg.bm, cfg.bn);
    }
}

}  // namespace onhip
