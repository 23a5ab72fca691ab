// Attention of one (batch, head) in one launch: scores = q k^T (* scale), Softmax over the keys, context = scores v,
// i.e. the chain MatMul -> [Mul] -> Softmax -> MatMul of a transformer block (device/x86/MatMul/mat_mul.c:10-102,
// device/x86/Softmax/softmax.c:26-59) with the head split and merge Transposes (device/x86/Transpose/transpose.c)
// folded into the operands' strides.  The scores never leave the registers.
//
// A workgroup of four wavefronts takes 64 queries of one (batch, head); k, then v of that head (at most 256 keys) sit
// in LDS.  A wavefront owns 16 queries and computes the TRANSPOSED scores S^T = k q^T with v_mfma_f32_16x16x4_f32:
// in the accumulator layout a lane then holds one query (column lane % 16) and, per 16-key tile, the 4 keys
// 4 (lane / 16) + r.  That makes
//   * the Softmax a reduction inside the lane (52 values for 197 keys) plus two exchanges between the lane quarters,
//   * the probabilities, as they lie in the registers, the B operand of the second product out^T = v^T P^T: MFMA step
//     (tile, r) reduces over exactly the four keys the lane quarters hold in register r, so P is never moved, and the
//     A operand is a row of v, a conflict-free LDS read.
// The first product's reduction index (the head dimension) may be enumerated in any order as long as both operands
// agree: a lane reads four consecutive channels 16 j + 4 (lane / 16) .. + 3 of its row with one 16-byte access and
// feeds them to four MFMA steps.
// 16-query wavefronts rather than 32-query ones: 197 tokens are 13 such units per head, 2496 for 64 images of 3 heads,
// which spread over the 1024 SIMDs in three rounds of a quarter of the 32-query unit's work each; 32-query units (7 per
// head, 1344) need two rounds of the full unit.
#include "igemm_kernel.hpp"

namespace onhip {

struct AttnParams {
    const float *q, *k, *v;
    float *o;
    long long qs[3], ks[3], vs[3], os[3];   // element strides of (batch, head, token); the head dimension is contiguous
    int heads, tokens, qblocks;   // qblocks: workgroups (64 queries each) per head
    float scale;
};

template <int NKT, int HD>
__global__ __launch_bounds__(256, 2) void attention_f32_kernel(const AttnParams p) {
    static_assert(HD % 16 == 0 && HD <= 64 && NKT >= 1 && NKT <= 16, "head dimension in 16s, at most 256 keys");
    constexpr int KEYS = NKT * 16;
    // floats per key row: 16-byte reads of 16 consecutive rows spread over 64 banks, and rows four apart (the lane
    // quarters of a step of the second product) start 16 banks apart
    constexpr int LD = HD + 4;
    constexpr int DT = HD / 16, QF = HD / 16;
    constexpr int PARTS = HD / 4, NV = (KEYS * PARTS + 255) / 256;
    // one buffer, first k, then v (fetched into registers while the scores are computed): two workgroups fit a compute unit
    __shared__ __attribute__((aligned(16))) float lds[KEYS * LD];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    // Workgroups are handed to the 8 XCDs round-robin and every XCD has an L2 of its own: renumber so that an XCD gets a
    // contiguous run of (head, query block) pairs and the query blocks of one head read k and v through one L2
    int qblock, bh;
    {
        const int nb = (int) gridDim.x, bid = (int) blockIdx.x;
        const int per = nb >> 3, rmd = nb & 7, xcd = bid & 7, idx = bid >> 3;
        const int lid = xcd * per + (xcd < rmd ? xcd : rmd) + idx;
        bh = lid / p.qblocks;
        qblock = lid - bh * p.qblocks;
    }
    const int b = bh / p.heads, h = bh - b * p.heads;
    const int T = p.tokens;
    // the launcher has checked that tokens * token stride stays below 2 GiB
    const rsrc_t rk = make_rsrc(p.k + b * p.ks[0] + h * p.ks[1], RSRC_RANGE);
    const rsrc_t rv = make_rsrc(p.v + b * p.vs[0] + h * p.vs[1], RSRC_RANGE);
    const unsigned kstride = (unsigned) p.ks[2] * 4, vstride = (unsigned) p.vs[2] * 4;

    // k of this head into LDS, rows past the last key as zeros
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int f = tid + i * 256;
        const int key = f / PARTS, part = f % PARTS;
        // buffer loads, rows past the last key at the out-of-range offset (zeros): no branch around a load, so the
        // compiler can count the loads in flight and wait for exactly the ones it needs
        const uint4 kk = buf_load_b128(rk, key < T ? (unsigned) key * kstride + part * 16 : OOB, 0);
        if ((i + 1) * 256 <= KEYS * PARTS || f < KEYS * PARTS) *reinterpret_cast<uint4 *>(lds + key * LD + part * 4) = kk;
    }
    // this lane's query row, the channels it feeds to the first product
    const int q0 = (qblock * 4 + wave) * 16;
    const int query = q0 + li;
    const bool active = q0 < T;   // uniform: a wavefront without queries only helps with the loads
    float4 qf[QF];
    {
        const float *qb = p.q + b * p.qs[0] + h * p.qs[1] + (long long) (query < T ? query : T - 1) * p.qs[2];
#pragma unroll
        for (int j = 0; j < QF; ++j) qf[j] = *reinterpret_cast<const float4 *>(qb + 16 * j + 4 * lg);   // rows past the last: unused
    }
    // v on its way into registers
    uint4 vreg[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int f = tid + i * 256;
        const int key = f / PARTS, part = f % PARTS;
        vreg[i] = buf_load_b128(rv, key < T ? (unsigned) key * vstride + part * 16 : OOB, 0);
    }
    __syncthreads();

    // S^T = k q^T: one accumulator per tile of 16 keys
    f32x4 s[NKT];
    if (active) {
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) s[t][r] = 0.0f;
#pragma unroll
        for (int j = 0; j < QF; ++j) {
            float4 kf[NKT];
#pragma unroll
            for (int t = 0; t < NKT; ++t) kf[t] = *reinterpret_cast<const float4 *>(lds + (16 * t + li) * LD + 16 * j + 4 * lg);
            // consecutive MFMAs go to different accumulators
#pragma unroll
            for (int t = 0; t < NKT; ++t) s[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t].x, qf[j].x, s[t], 0, 0, 0);
#pragma unroll
            for (int t = 0; t < NKT; ++t) s[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t].y, qf[j].y, s[t], 0, 0, 0);
#pragma unroll
            for (int t = 0; t < NKT; ++t) s[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t].z, qf[j].z, s[t], 0, 0, 0);
#pragma unroll
            for (int t = 0; t < NKT; ++t) s[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t].w, qf[j].w, s[t], 0, 0, 0);
        }

        // Softmax over the keys (softmax.c:26-59: subtract the row maximum, exponential, divide by the sum); keys past the
        // last count as minus infinity.  exp(x) as exp2(x log2 e) with the hardware's exp2: within 1e-5 of expf here
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = 16 * t + 4 * lg + r;
                const float val = key < T ? __fmul_rn(s[t][r], p.scale) : -INFINITY;
                s[t][r] = val;
                mx = fmaxf(mx, val);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = __builtin_amdgcn_exp2f(__fmul_rn(__fsub_rn(s[t][r], mx), 1.44269504088896340736f));
                s[t][r] = e;
                sum += e;
            }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) s[t][r] = __fmul_rn(s[t][r], inv);
    }

    // everybody is done with k: v takes its place
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int f = tid + i * 256;
        const int key = f / PARTS, part = f % PARTS;
        if ((i + 1) * 256 <= KEYS * PARTS || f < KEYS * PARTS) *reinterpret_cast<uint4 *>(lds + key * LD + part * 4) = vreg[i];
    }
    __syncthreads();
    if (!active) return;

    // out^T = v^T P^T: step (t, r) reduces over the keys the four lane quarters hold in register r of tile t (rows past
    // the last key hold zeros in v and zero probabilities).  Row m of output tile d stands for channel DT m + d, so a lane
    // reads the A operands of a step's DT products, v[key][DT li .. + DT - 1], with one access, and ends up with the
    // 4 DT consecutive channels from 4 DT (lane / 16) of its query.  No step is skipped at run time: a branch per
    // step would end the block the LDS reads are scheduled in, and their latency would show once per step.
    typedef float vrow_t __attribute__((ext_vector_type(DT)));
    f32x4 o[DT];
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[d][r] = 0.0f;
    vrow_t va[2][4];   // the operands of the next tile are read while this tile's products run
#pragma unroll
    for (int r = 0; r < 4; ++r) va[0][r] = *reinterpret_cast<const vrow_t *>(lds + (4 * lg + r) * LD + DT * li);
#pragma unroll
    for (int t = 0; t < NKT; ++t) {
        if (t + 1 < NKT) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                va[(t + 1) & 1][r] = *reinterpret_cast<const vrow_t *>(lds + (16 * (t + 1) + 4 * lg + r) * LD + DT * li);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int d = 0; d < DT; ++d)
                o[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(va[t & 1][r][d], s[t][r], o[d], 0, 0, 0);
    }

    if (query < T) {
        float *ob = p.o + b * p.os[0] + h * p.os[1] + (long long) query * p.os[2] + 4 * DT * lg;
        float vals[4 * DT];
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
            for (int r = 0; r < 4; ++r) vals[DT * r + d] = o[d][r];
#pragma unroll
        for (int i = 0; i < DT; ++i)
            *reinterpret_cast<float4 *>(ob + 4 * i) = make_float4(vals[4 * i], vals[4 * i + 1], vals[4 * i + 2], vals[4 * i + 3]);
    }
}

template <int NKT, int HD>
static int attention_launch_one(const AttnParams &p, int batch, hipStream_t stream) {
    const dim3 grid((unsigned) (p.qblocks * batch * p.heads));
    hipLaunchKernelGGL((attention_f32_kernel<NKT, HD>), grid, dim3(256), 0, stream, p);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

template <int HD>
static int attention_launch_hd(const AttnParams &p, int batch, hipStream_t stream) {
    const int nkt = (p.tokens + 15) / 16;
    if (nkt <= 4) return attention_launch_one<4, HD>(p, batch, stream);
    if (nkt <= 7) return attention_launch_one<7, HD>(p, batch, stream);
    if (nkt <= 10) return attention_launch_one<10, HD>(p, batch, stream);
    if (nkt <= 13) return attention_launch_one<13, HD>(p, batch, stream);
    return attention_launch_one<16, HD>(p, batch, stream);
}

int attention_f32_launch(const onhip_attention_desc_t &d, const float *q, const float *k, const float *v, float *out,
                         hipStream_t stream) {
    AttnParams p;
    p.q = q; p.k = k; p.v = v; p.o = out;
    for (int i = 0; i < 3; ++i) {
        p.qs[i] = d.q_strides[i]; p.ks[i] = d.k_strides[i]; p.vs[i] = d.v_strides[i]; p.os[i] = d.out_strides[i];
    }
    p.heads = d.heads;
    p.tokens = d.tokens;
    p.qblocks = (d.tokens + 63) / 64;
    p.scale = d.scale;
    // k and v are read through 32-bit byte offsets from the head's first row
    if (d.tokens * d.k_strides[2] * 4 >= (1LL << 31) || d.tokens * d.v_strides[2] * 4 >= (1LL << 31))
        return set_error(ONHIP_ERR_ARG, "attention: tokens x token stride of k or v reaches 2 GiB");
    if (d.head_dim == 64) return attention_launch_hd<64>(p, d.batch, stream);
    return attention_launch_hd<32>(p, d.batch, stream);
}

}  // namespace onhip
