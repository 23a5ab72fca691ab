// Implicit GEMM for operands whose K runs contiguously in memory (NHWC int8 activations against tap-major packed
// int8 weights): operand tiles go from global memory straight into LDS (buffer_load ... lds, 16 bytes per lane, no
// register hop and no LDS store instruction), through a ring of NST stage buffers, and the K loop is nothing but LDS
// reads at fixed addresses and MFMAs.
//
//   * a stage is KS bytes of K (128 or 64) for every row of the BM x BN tile: one wave-wide load covers 1024 / KS
//     rows, the lanes of a row taking its 16-byte units, so a load reads whole cache lines;
//   * LDS keeps a stage row-major ([row][KS bytes]); an MFMA step wants unit 2s + (lane / 32) of row lane % 32, a
//     stride of KS bytes between lanes.  A load cannot choose where its bytes land in LDS (lane l at +16 l), but it can
//     choose which global unit a lane fetches: slot c of row r holds unit c ^ swz(r), and the reader asks for slot
//     u ^ swz(r).  swz spreads 16 consecutive rows over the 16 bank groups of 16 bytes (no bank conflicts measured);
//   * stage buffers are compile-time offsets in the instruction's immediate (the loop is unrolled over the ring), the
//     per-lane addresses of every K step of a stage are computed once, so the loop has no address arithmetic;
//   * the LDS reads are inline assembly: to the compiler a read of LDS may alias a load-to-LDS still in flight, and it
//     would wait for all of them (vmcnt(0)) before every read, which undoes the ring.  Waits are placed by hand:
//     vmcnt((NST - 2) * loads per stage) before the one barrier of a stage, lgkmcnt per K step.
//
// Requirements (dma_ok): K-vector loader, at most 64 taps, no split-K, and either a whole number of stages per filter tap
// (channel pitch in bytes a multiple of KS) or, int8 only (MULTI), taps of 16 or 32 bytes: a 64-byte stage then holds
// four or two taps, the tap is a per-lane quantity, and the last stage may reach past the end of K (the weights it reads
// there meet activations that are zero).  Everything else runs igemm_kernel.  The accumulator layout is that of
// igemm_kernel, and so are the epilogues (write_tile, write_tile_nhwc_s8): same bits.
//
// Replaces, like igemm_kernel's int8 variant: the int32 GEMM and de-quantisation of device/x86/Conv/conv.c:1024-1056.
#pragma once
#include "igemm_kernel.hpp"

namespace onhip {

typedef __attribute__((address_space(3))) void *lds_ptr_t;

#if defined(__HIP_DEVICE_COMPILE__)
template <int OFF>
__device__ __forceinline__ i32x4 lds_read_b128(unsigned addr) {
    i32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    return v;
}

// waits until at most CNT LDS reads are outstanding and ties the operand registers of the step about to be multiplied
// to that wait, so that no MFMA reading them is scheduled before it
template <int CNT, int TM, int TN>
__device__ __forceinline__ void wait_operands(i32x4 (&av)[TM], i32x4 (&bv)[TN]) {
    static_assert(TM >= 1 && TM <= 2 && TN >= 1 && TN <= 2, "operand lists below");
    if constexpr (TM == 2 && TN == 2) asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(av[0]), "+v"(av[1]), "+v"(bv[0]), "+v"(bv[1]) : "n"(CNT) : "memory");
    else if constexpr (TM == 1 && TN == 2) asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(av[0]), "+v"(bv[0]), "+v"(bv[1]) : "n"(CNT) : "memory");
    else if constexpr (TM == 2 && TN == 1) asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(av[0]), "+v"(av[1]), "+v"(bv[0]) : "n"(CNT) : "memory");
    else asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(av[0]), "+v"(bv[0]) : "n"(CNT) : "memory");
}
#endif

template <int KS> __device__ __forceinline__ int dma_swz(int row) { return KS == 128 ? ((row >> 1) & 7) : ((row >> 2) & 3); }

template <int DT, int BM, int BN, int WM, int WN, int KS, int NST, bool MULTI = false>
__global__ __launch_bounds__(THREADS) void igemm_dma_kernel(const IgemmParams p) {
    // device pass only: the host pass cannot parse the inline assembly's register constraints, and a kernel whose body it
    // rejects gets no launch stub
#if defined(__HIP_DEVICE_COMPILE__)
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    static_assert(DT == DT_I8 || DT == DT_BF16 || DT == DT_F16, "operand types stored as 16-byte vectors of K");
    // MULTI: a filter tap is shorter than a stage (16 or 32 bytes of K: up to 16 or 32 int8 channels), so a 64-byte stage
    // holds four or two taps and the tap is a per-lane quantity, a function of the unit the lane fetches
    static_assert(!MULTI || (DT == DT_I8 && KS == 64), "several taps per stage: int8, 64-byte stages");
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int SLOTS = KS / 16, KSTEPS = SLOTS / 2;
    constexpr int ROWS_PER_LOAD = 1024 / KS;
    constexpr int A_LOADS = BM / ROWS_PER_LOAD / 4, B_LOADS = BN / ROWS_PER_LOAD / 4;   // per wavefront and stage
    static_assert(A_LOADS >= 1 && B_LOADS >= 1, "every wavefront loads part of both operands");
    constexpr int STAGE = (BM + BN) * KS, PER_STAGE = A_LOADS + B_LOADS;
    // a ds_read reaches 64 KiB beyond its address register: a ring longer than that gets one set of read addresses per
    // 64 KiB window, and a stage's offset inside its window is the instruction's immediate
    static_assert(NST >= 2 && NST * STAGE <= 160 * 1024, "the ring must fit the 160 KiB of LDS of a compute unit");
    constexpr int NSETS = (NST * STAGE + 65535) / 65536;
    // after the K loop the same memory holds the store's staging area, the quantised activation table and the per-row constants
    constexpr int OUT_STAGE = DT == DT_I8 ? BN * (BM + 16) : BN * (2 * BM + 16), ROWS_AT = OUT_STAGE + (DT == DT_I8 ? 8192 : 16384), OUT_BYTES = ROWS_AT + 2 * BM * 4;
    static_assert(ROWS_AT % 16 == 0, "the per-row constants are read 16 bytes at a time");
    constexpr int LDS_BYTES = NST * STAGE > OUT_BYTES ? NST * STAGE : OUT_BYTES;
    __shared__ __attribute__((aligned(1024))) unsigned char lds[LDS_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;
    // XCD-aware tile order, as igemm_kernel: every XCD gets a contiguous run of tiles
    const int tiles_m = (p.M + BM - 1) / BM;
    int lid;
    {
        const int bid = blockIdx.x, nb = (int) gridDim.x;
        const int q = nb >> 3, rmd = nb & 7, xcd = bid & 7, idx = bid >> 3;
        lid = xcd * q + (xcd < rmd ? xcd : rmd) + idx;
    }
    const int tile_n = (int) div31((unsigned) lid, p.div_tiles_m), tile_m = lid - tile_n * tiles_m;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    // the per-row constants of the epilogue, one row per thread, fetched while the first stages are on their way: the
    // de-quantisation factor weight_aux / 127 (conv.c:1049-1056) and the int32 bias as a float
    // (the 16-bit types have the fp32 bias alone)
    float row_coeff = 0.0f, row_bias = 0.0f;
    if (tid < BM) {
        const int m = m0 + tid;
        if constexpr (DT == DT_I8) {
            const rsrc_t raux = make_rsrc(p.weight_aux, (unsigned) (p.M * 4));
            const rsrc_t rb32 = make_rsrc(p.bias32, p.bias32 ? (unsigned) (p.M * 4) : 0u);
            row_coeff = buf_load_f32(raux, (unsigned) m * 4u, 0);          // rows beyond M read as zero
            row_bias = (float) (int) __builtin_amdgcn_raw_buffer_load_b32(rb32, (unsigned) m * 4u, 0, 0);
        } else {
            const rsrc_t rb = make_rsrc(p.bias, p.bias_mode == BIAS_M ? (unsigned) (p.M * 4) : 0u);
            row_bias = buf_load_f32(rb, (unsigned) m * 4u, 0);
        }
    }

    // the quantised activation table that the int8 NHWC store gathers from (8 KiB, 32 bytes per thread): requested here,
    // before any operand load (being the oldest loads in flight, the K loop's counted waits cover them), and written
    // to LDS behind the staging area once the K loop has left it, instead of a memory round trip plus a barrier of its own
    // at the head of every tile's store
    uint4 table_q[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
    bool table_pre = false;
    if constexpr (DT == DT_I8) {
        table_pre = p.out_s8 && p.out_mode == OUT_PLAIN && p.c_stride_m == 1 && !p.acc_out && p.ep.qlut != nullptr &&
                    (p.ep.act == SILU || p.ep.act == ONHIP_ACT_GELU_LUT);   // uniform
        if (table_pre) {
            const rsrc_t rq = make_rsrc(p.ep.qlut, 8192u);
            table_q[0] = buf_load_b128(rq, (unsigned) tid * 16u, 0);
            table_q[1] = buf_load_b128(rq, (unsigned) (tid + THREADS) * 16u, 0);
        }
    }
    asm volatile("" ::: "memory");   // these loads stay ahead of the operand loads: the stage waits count loads in issue order

    const char *a_base = reinterpret_cast<const char *>(p.A);
    const char *b_base = reinterpret_cast<const char *>(p.B) - (size_t) p.b_shift_bytes;
    const unsigned a_bytes = (unsigned) p.a_slice_bytes, b_bytes = (unsigned) (p.b_slice_bytes + p.b_shift_bytes);
    const int k_stages = MULTI ? (p.k_units + SLOTS - 1) / SLOTS : p.k_units / SLOTS;   // MULTI: the last stage may be ragged
    const int stages_per_tap = MULTI ? 1 : p.units_per_tap / SLOTS;

    // this lane's share of a wave-wide load: row lane / SLOTS of the load's rows, slot lane % SLOTS, which holds the
    // row's unit slot ^ swz(row)
    const int lrow = lane / SLOTS, lslot = lane % SLOTS;
    unsigned a_voff[A_LOADS], b_voff[B_LOADS], b_mask_lo[B_LOADS], b_mask_hi[B_LOADS];
    unsigned b_tap_sub[MULTI ? B_LOADS : 1], b_within[MULTI ? B_LOADS : 1];   // MULTI: tap within the stage, byte offset within the tap
#pragma unroll
    for (int t = 0; t < A_LOADS; ++t) {
        const int row = (wave * A_LOADS + t) * ROWS_PER_LOAD + lrow;
        const int m = m0 + row;
        a_voff[t] = m < p.M ? (unsigned) (m * p.lda + ((lslot ^ dma_swz<KS>(row)) * 16)) : OOB;
    }
#pragma unroll
    for (int t = 0; t < B_LOADS; ++t) {
        const int row = (wave * B_LOADS + t) * ROWS_PER_LOAD + lrow;
        const ColState c = make_col<BL_KVEC>(p, n0 + row);
        const int unit = lslot ^ dma_swz<KS>(row);
        if constexpr (MULTI) {
            b_voff[t] = c.pixoff;
            b_tap_sub[t] = (unsigned) unit / (unsigned) p.units_per_tap;      // units_per_tap is 1 or 2
            b_within[t] = ((unsigned) unit % (unsigned) p.units_per_tap) * 16u;
        } else {
            b_voff[t] = c.pixoff == OOB ? OOB : c.pixoff + (unsigned) (unit * 16);
        }
        b_mask_lo[t] = c.mask_lo;
        b_mask_hi[t] = c.mask_hi;
    }
    // Stages are issued in ascending order, one call each, so the filter tap of the next stage to load is running scalar
    // state: a stage lies inside one tap (dma_ok), whose offset in the image and bit in the lanes' masks are uniform.
    int next_in_tap = 0;
    unsigned next_tap = 0, next_ti = 0, next_tj = 0;
    auto issue = [&](int kt, int buf) __attribute__((always_inline)) {   // buf == kt % NST, a constant where it is called
        const bool live = kt < k_stages;
        const rsrc_t ra = make_rsrc(a_base, live ? a_bytes : 0u);
        const rsrc_t rb = make_rsrc(b_base, live ? b_bytes : 0u);
        unsigned char *base = lds + buf * STAGE;
        const unsigned b_soff = (next_ti * (unsigned) p.W + next_tj) * (unsigned) p.pix_stride + (unsigned) (next_in_tap * KS);
        const unsigned bitpos = next_tap & 31u;
        const bool hi = next_tap >= 32u;
#pragma unroll
        for (int t = 0; t < A_LOADS; ++t)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t) (base + (wave * A_LOADS + t) * 1024), 16, a_voff[t],
                                                     (unsigned) (kt * KS), 0, 0);
        if constexpr (MULTI) {
            const unsigned taps_per_stage = (unsigned) SLOTS / (unsigned) p.units_per_tap;
#pragma unroll
            for (int t = 0; t < B_LOADS; ++t) {
                const unsigned tap = (unsigned) kt * taps_per_stage + b_tap_sub[t];
                const unsigned ti = fast_div(tap, p.magic_kw, p.pass_kw), tj = tap - ti * (unsigned) p.kw;
                const unsigned word = tap >= 32u ? b_mask_hi[t] : b_mask_lo[t];
                const bool in = live && tap < (unsigned) p.khkw && ((word >> (tap & 31u)) & 1u) != 0u && b_voff[t] != OOB;
                const unsigned voff = in ? b_voff[t] + (ti * (unsigned) p.W + tj) * (unsigned) p.pix_stride + b_within[t] : OOB;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t) (base + BM * KS + (wave * B_LOADS + t) * 1024), 16, voff, 0, 0, 0);
            }
            return;
        }
#pragma unroll
        for (int t = 0; t < B_LOADS; ++t) {
            // the tap's bit of the lane's validity mask as a bit field, the choice between the pixel and "outside" as bit
            // arithmetic: four vector instructions, no compare, no branch (a 1x1 filter has bit 0 set for every pixel)
            const unsigned word = hi ? b_mask_hi[t] : b_mask_lo[t];
            const unsigned keep = 0u - __builtin_amdgcn_ubfe(word, bitpos, 1u);   // all ones when the tap lies inside the image
            const unsigned voff = (b_voff[t] & keep) | (OOB & ~keep);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t) (base + BM * KS + (wave * B_LOADS + t) * 1024), 16, voff, b_soff, 0, 0);
        }
        if (++next_in_tap == stages_per_tap) {
            next_in_tap = 0;
            ++next_tap;
            if (++next_tj == (unsigned) p.kw) { next_tj = 0; ++next_ti; }
        }
    };

    typename Traits<DT>::acc_t acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;

#pragma unroll
    for (int s = 0; s < NST - 1; ++s) issue(s, s);

    const unsigned lds0 = (unsigned) (size_t) (__attribute__((address_space(3))) unsigned char *) lds;
    unsigned a_addr[NSETS][TM][KSTEPS], b_addr[NSETS][TN][KSTEPS];
#pragma unroll
    for (int w = 0; w < NSETS; ++w) {
#pragma unroll
        for (int a = 0; a < TM; ++a) {
            const int row = wm * TM * 32 + a * 32 + li;
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) a_addr[w][a][s] = lds0 + w * 65536 + row * KS + (((2 * s + lh) ^ dma_swz<KS>(row)) * 16);
        }
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int row = wn * TN * 32 + b * 32 + li;
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s)
                b_addr[w][b][s] = lds0 + w * 65536 + BM * KS + row * KS + (((2 * s + lh) ^ dma_swz<KS>(row)) * 16);
        }
    }

    auto stage_body = [&](int kt, auto bufc) __attribute__((always_inline)) {
        constexpr int SET = (decltype(bufc)::value * STAGE) >> 16, SB = (decltype(bufc)::value * STAGE) & 0xffff;
        // this wavefront's loads of stage kt have landed once at most the loads of the NST - 2 later stages are out;
        // the barrier says the same of everybody's, and that everybody has read stage kt - 1, whose buffer is loaded next
        asm volatile("s_waitcnt vmcnt(%0)" :: "n"((NST - 2) * PER_STAGE) : "memory");
        __builtin_amdgcn_s_barrier();
        i32x4 av[2][TM], bv[2][TN];
#pragma unroll
        for (int a = 0; a < TM; ++a) av[0][a] = lds_read_b128<SB>(a_addr[SET][a][0]);
#pragma unroll
        for (int b = 0; b < TN; ++b) bv[0][b] = lds_read_b128<SB>(b_addr[SET][b][0]);
        issue(kt + NST - 1, (decltype(bufc)::value + NST - 1) % NST);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            const int cur = s & 1, nxt = cur ^ 1;
            if (s + 1 < KSTEPS) {
#pragma unroll
                for (int a = 0; a < TM; ++a) av[nxt][a] = lds_read_b128<SB>(a_addr[SET][a][s + 1]);
#pragma unroll
                for (int b = 0; b < TN; ++b) bv[nxt][b] = lds_read_b128<SB>(b_addr[SET][b][s + 1]);
                wait_operands<TM + TN>(av[cur], bv[cur]);
            } else {
                wait_operands<0>(av[cur], bv[cur]);
            }
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int b = 0; b < TN; ++b) {
                    if constexpr (DT == DT_I8)
                        acc[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av[cur][a], bv[cur][b], acc[a][b], 0, 0, 0);
                    else if constexpr (DT == DT_BF16)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av[cur][a]),
                                                                            __builtin_bit_cast(bf16x8, bv[cur][b]), acc[a][b], 0, 0, 0);
                    else
                        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, av[cur][a]),
                                                                           __builtin_bit_cast(f16x8, bv[cur][b]), acc[a][b], 0, 0, 0);
                }
        }
    };
    int kt = 0;
    for (; kt + NST <= k_stages; kt += NST) {
        [&]<int... J>(std::integer_sequence<int, J...>) __attribute__((always_inline)) {
            (stage_body(kt + J, std::integral_constant<int, J>{}), ...);
        }(std::make_integer_sequence<int, NST>{});
    }
    [&]<int... J>(std::integer_sequence<int, J...>) __attribute__((always_inline)) {
        ((kt + J < k_stages ? stage_body(kt + J, std::integral_constant<int, J>{}) : (void) 0), ...);
    }(std::make_integer_sequence<int, NST>{});

    // the loads issued past the end carry empty descriptors but still write (zeros) into LDS: they have to be home, and
    // every wavefront done with the operand buffers, before the store reuses that memory
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    float *rows = reinterpret_cast<float *>(lds + ROWS_AT);
    if (tid < BM) {
        if constexpr (DT == DT_I8) {
            rows[tid] = __fdiv_rn(row_coeff, 127.0f);
            rows[BM + tid] = row_bias;
        } else {
            rows[tid] = row_bias;
        }
    }
    if constexpr (DT == DT_I8) {
        if (table_pre) {
            unsigned char *ql = lds + BN * (BM + 16);   // where write_tile_nhwc_s8 looks for it
            reinterpret_cast<uint4 *>(ql)[tid] = table_q[0];
            reinterpret_cast<uint4 *>(ql)[tid + THREADS] = table_q[1];
            if (tid == 0) ql[-1] = 0;                   // its "below the table" entry
        }
    }
    __syncthreads();

    const int m_wave = m0 + wm * (BM / WM), n_wave = n0 + wn * (BN / WN);
    if constexpr (DT == DT_I8) {
        if (p.out_s8 && p.out_mode == OUT_PLAIN && p.c_stride_m == 1 && !p.acc_out) {
            switch (p.ep.act) {
                case NOT_ACT:
                case RELU6: write_tile_nhwc_s8<EPI_NONE, BM, BN, TM, TN, true>(p, acc, lds, m0, n0, m_wave, n_wave, li, lh, tid, rows, table_pre); break;
                case RELU: write_tile_nhwc_s8<EPI_RELU, BM, BN, TM, TN, true>(p, acc, lds, m0, n0, m_wave, n_wave, li, lh, tid, rows, table_pre); break;
                case CLIP: write_tile_nhwc_s8<EPI_CLIP, BM, BN, TM, TN, true>(p, acc, lds, m0, n0, m_wave, n_wave, li, lh, tid, rows, table_pre); break;
                case SILU:
                case ONHIP_ACT_GELU_LUT: write_tile_nhwc_s8<EPI_LUT, BM, BN, TM, TN, true>(p, acc, lds, m0, n0, m_wave, n_wave, li, lh, tid, rows, table_pre); break;
                default: write_tile_nhwc_s8<EPI_GENERIC, BM, BN, TM, TN, true>(p, acc, lds, m0, n0, m_wave, n_wave, li, lh, tid, rows, table_pre); break;
            }
            return;
        }
    } else {
        if (p.out_h16) {
            switch (p.ep.act) {
                case NOT_ACT:
                case RELU6: write_tile_nhwc_h16<DT, EPI_NONE, BM, BN, TM, TN>(p, acc, lds, m0, n0, m_wave, n_wave, li, lh, tid, rows); break;
                case RELU: write_tile_nhwc_h16<DT, EPI_RELU, BM, BN, TM, TN>(p, acc, lds, m0, n0, m_wave, n_wave, li, lh, tid, rows); break;
                case CLIP: write_tile_nhwc_h16<DT, EPI_CLIP, BM, BN, TM, TN>(p, acc, lds, m0, n0, m_wave, n_wave, li, lh, tid, rows); break;
                case SILU:
                case ONHIP_ACT_GELU_LUT: write_tile_nhwc_h16<DT, EPI_LUT, BM, BN, TM, TN>(p, acc, lds, m0, n0, m_wave, n_wave, li, lh, tid, rows); break;
                default: write_tile_nhwc_h16<DT, EPI_GENERIC, BM, BN, TM, TN>(p, acc, lds, m0, n0, m_wave, n_wave, li, lh, tid, rows); break;
            }
            return;
        }
    }
    switch (p.ep.act) {
        case NOT_ACT:
        case RELU6: write_tile<DT, EPI_NONE, TM, TN, false, DT == DT_I8>(p, acc, 0, m_wave, n_wave, li, lh, rows + (m_wave - m0), rows + BM + (m_wave - m0)); break;
        case RELU: write_tile<DT, EPI_RELU, TM, TN, false, DT == DT_I8>(p, acc, 0, m_wave, n_wave, li, lh, rows + (m_wave - m0), rows + BM + (m_wave - m0)); break;
        case CLIP: write_tile<DT, EPI_CLIP, TM, TN, false, DT == DT_I8>(p, acc, 0, m_wave, n_wave, li, lh, rows + (m_wave - m0), rows + BM + (m_wave - m0)); break;
        case SILU:
        case ONHIP_ACT_GELU_LUT: write_tile<DT, EPI_LUT, TM, TN, false, DT == DT_I8>(p, acc, 0, m_wave, n_wave, li, lh, rows + (m_wave - m0), rows + BM + (m_wave - m0)); break;
        default: write_tile<DT, EPI_GENERIC, TM, TN, false, DT == DT_I8>(p, acc, 0, m_wave, n_wave, li, lh, rows + (m_wave - m0), rows + BM + (m_wave - m0)); break;
    }
#endif
}

// bytes of K per stage this problem can run with (128, 64) or 0: whole stages per filter tap
inline int dma_stage_bytes(const IgemmParams &p) {
    const int tap_bytes = p.units_per_tap * 16;
    return tap_bytes % 128 == 0 ? 128 : tap_bytes % 64 == 0 ? 64 : 0;
}
// int8 with 16 or 32 bytes of K per filter tap (up to 16 / 32 channels): 64-byte stages that hold four or two taps
inline bool dma_multi_tap(int dtype, const IgemmParams &p) {
    return dtype == DT_I8 && (p.units_per_tap == 1 || p.units_per_tap == 2) && p.khkw <= 64;
}

template <int DT, int BM, int BN, int KS, int NST, bool MULTI = false>
int dma_launch_one(const IgemmParams &p_in, hipStream_t stream) {
    IgemmParams p = p_in;
    const int tiles_m = (p.M + BM - 1) / BM;
    const long long tiles = (long long) tiles_m * ((p.N + BN - 1) / BN);
    if (tiles > 0x7fffffffLL) return set_error(ONHIP_ERR_ARG, "igemm: too many tiles");
    p.div_ohw = make_div31((unsigned) (p.OHW > 0 ? p.OHW : 1));
    p.div_ow = make_div31((unsigned) (p.OW > 0 ? p.OW : 1));
    p.div_tiles_m = make_div31((unsigned) tiles_m);
    hipLaunchKernelGGL((igemm_dma_kernel<DT, BM, BN, 2, 2, KS, NST, MULTI>), dim3((unsigned) tiles), dim3(THREADS), 0, stream, p);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

template <int DT>
int dma_launch_dt(const IgemmLaunch &cfg, const IgemmParams &p, hipStream_t stream) {
    const int key = cfg.bm * 1000 + cfg.bn;
    if constexpr (DT == DT_I8) {
        if (dma_multi_tap(DT, p)) {   // short taps: one ring length
            switch (key) {
                case 128128: return dma_launch_one<DT, 128, 128, 64, 3, true>(p, stream);
                case 128064: return dma_launch_one<DT, 128, 64, 64, 4, true>(p, stream);
                case 64128: return dma_launch_one<DT, 64, 128, 64, 4, true>(p, stream);
                case 64064: return dma_launch_one<DT, 64, 64, 64, 4, true>(p, stream);
            }
            return set_error(ONHIP_ERR_ARG, "igemm: no direct-to-LDS kernel for tile %dx%d", cfg.bm, cfg.bn);
        }
    }
    const int ks = dma_stage_bytes(p);
    // cfg.ring != 0: the long rings, more than 64 KiB of LDS for one workgroup (one or two workgroups per compute unit,
    // three to seven stages of loads in flight each); otherwise rings of at most 64 KiB
    if (ks == 128) {
        switch (key + (cfg.ring ? 1000000 : 0)) {
            case 128128: return dma_launch_one<DT, 128, 128, 128, 2>(p, stream);
            case 128064: return dma_launch_one<DT, 128, 64, 128, 2>(p, stream);
            case 64128: return dma_launch_one<DT, 64, 128, 128, 2>(p, stream);
            case 64064: return dma_launch_one<DT, 64, 64, 128, 3>(p, stream);
            case 1128128: return dma_launch_one<DT, 128, 128, 128, 4>(p, stream);
            case 1128064: return dma_launch_one<DT, 128, 64, 128, 5>(p, stream);
            case 1064128: return dma_launch_one<DT, 64, 128, 128, 5>(p, stream);
            case 1064064: return dma_launch_one<DT, 64, 64, 128, 5>(p, stream);
        }
    } else {
        switch (key + (cfg.ring ? 1000000 : 0)) {
            case 128128: return dma_launch_one<DT, 128, 128, 64, 3>(p, stream);
            case 128064: return dma_launch_one<DT, 128, 64, 64, 4>(p, stream);
            case 64128: return dma_launch_one<DT, 64, 128, 64, 4>(p, stream);
            case 64064: return dma_launch_one<DT, 64, 64, 64, 4>(p, stream);
            case 1128128: return dma_launch_one<DT, 128, 128, 64, 6>(p, stream);
            case 1128064: return dma_launch_one<DT, 128, 64, 64, 8>(p, stream);
            case 1064128: return dma_launch_one<DT, 64, 128, 64, 8>(p, stream);
            case 1064064: return dma_launch_one<DT, 64, 64, 64, 8>(p, stream);
        }
    }
    return set_error(ONHIP_ERR_ARG, "igemm: no direct-to-LDS kernel for tile %dx%d", cfg.bm, cfg.bn);
}

}  // namespace onhip
