// Attention of one (batch, head) in one launch: scores = q k^T (* scale), Softmax over the keys, context = scores v,
// i.e. the chain MatMul -> [Mul] -> Softmax -> MatMul of a transformer block (device/x86/MatMul/mat_mul.c:10-102,
// device/x86/Softmax/softmax.c:26-59) with the head split and merge Transposes (device/x86/Transpose/transpose.c)
// folded into the operands' strides.  The scores never leave the registers.
//
// A workgroup of four wavefronts takes 128 queries of one (batch, head); k, then v of that head (at most 256 keys) sit
// in LDS.  A wavefront owns 32 queries and computes the TRANSPOSED scores S^T = k q^T with v_mfma_f32_32x32x2_f32:
// in the accumulator layout a lane then holds one query (column lane % 32) and, per 32-key tile, the 16 keys
// 8 (r / 4) + 4 (lane / 32) + r % 4.  That makes
//   * the Softmax a reduction inside the lane (112 values for 197 keys) plus one exchange between the lane halves,
//   * the probabilities, as they lie in the registers, the B operand of the second product out^T = v^T P^T: MFMA step
//     (tile, r) reduces over exactly the key pair the two lane halves hold in register r, so P is never moved, and the
//     A operand is v[key][channel lane % 32], a conflict-free LDS read.
// The first product's reduction index (the head dimension) may be enumerated in any order as long as both operands
// agree: a lane reads four consecutive channels 8 j + 4 (lane / 32) .. + 3 of its row with one 16-byte access and
// feeds them to four MFMA steps.
#include "igemm_kernel.hpp"

namespace onhip {

struct AttnParams {
    const float *q, *k, *v;
    float *o;
    long long qs[3], ks[3], vs[3], os[3];   // element strides of (batch, head, token); the head dimension is contiguous
    int heads, tokens;
    float scale;
};

template <int NKT, int HD>
__global__ __launch_bounds__(256, (NKT * HD >= 512 ? 1 : 2)) void attention_f32_kernel(const AttnParams p) {
    static_assert(HD % 32 == 0 && HD <= 128 && NKT >= 1 && NKT <= 8, "head dimension in 32s, at most 256 keys");
    constexpr int KEYS = NKT * 32;
    constexpr int LDK = HD + 4;    // floats per key row of k: 16-byte reads of 32 consecutive rows spread over all banks
    constexpr int LDV = HD + 8;    // of v: rows four apart (the two lane halves of a step) fall into different bank halves
    constexpr int DT = HD / 32, QF = HD / 8;
    constexpr int PARTS = HD / 4, NV = (KEYS * PARTS + 255) / 256;
    // one buffer, first k, then v (fetched into registers while the scores are computed): two workgroups fit a compute unit
    __shared__ __attribute__((aligned(16))) float lds[KEYS * LDV];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int bh = blockIdx.y, b = bh / p.heads, h = bh - b * p.heads;
    const int T = p.tokens;
    const float *kb = p.k + b * p.ks[0] + h * p.ks[1];
    const float *vb = p.v + b * p.vs[0] + h * p.vs[1];

    // k of this head into LDS, rows past the last key as zeros
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int f = tid + i * 256;
        const int key = f / PARTS, part = f % PARTS;
        float4 kk = make_float4(0.f, 0.f, 0.f, 0.f);
        if (key < T) kk = *reinterpret_cast<const float4 *>(kb + key * p.ks[2] + part * 4);
        if (f < KEYS * PARTS) *reinterpret_cast<float4 *>(lds + key * LDK + part * 4) = kk;
    }
    // this lane's query row, the channels it feeds to the first product
    const int q0 = (blockIdx.x * 4 + wave) * 32;
    const int query = q0 + li;
    const bool active = q0 < T;   // uniform: a wavefront without queries only helps with the loads
    float4 qf[QF];
    {
        const float *qb = p.q + b * p.qs[0] + h * p.qs[1] + (long long) query * p.qs[2];
#pragma unroll
        for (int j = 0; j < QF; ++j)
            qf[j] = query < T ? *reinterpret_cast<const float4 *>(qb + 8 * j + 4 * lh) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    // v on its way into registers
    float4 vreg[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int f = tid + i * 256;
        const int key = f / PARTS, part = f % PARTS;
        vreg[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (key < T) vreg[i] = *reinterpret_cast<const float4 *>(vb + key * p.vs[2] + part * 4);
    }
    __syncthreads();

    // S^T = k q^T: one accumulator per tile of 32 keys
    f32x16 s[NKT];
    if (active) {
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[t][r] = 0.0f;
#pragma unroll
        for (int j = 0; j < QF; ++j) {
            float4 kf[NKT];
#pragma unroll
            for (int t = 0; t < NKT; ++t) kf[t] = *reinterpret_cast<const float4 *>(lds + (32 * t + li) * LDK + 8 * j + 4 * lh);
            // consecutive MFMAs go to different accumulators
#pragma unroll
            for (int t = 0; t < NKT; ++t) s[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[t].x, qf[j].x, s[t], 0, 0, 0);
#pragma unroll
            for (int t = 0; t < NKT; ++t) s[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[t].y, qf[j].y, s[t], 0, 0, 0);
#pragma unroll
            for (int t = 0; t < NKT; ++t) s[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[t].z, qf[j].z, s[t], 0, 0, 0);
#pragma unroll
            for (int t = 0; t < NKT; ++t) s[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[t].w, qf[j].w, s[t], 0, 0, 0);
        }

        // Softmax over the keys (softmax.c:26-59: subtract the row maximum, exponential, divide by the sum); keys past the
        // last count as minus infinity.  exp(x) as exp2(x log2 e) with the hardware's exp2: within 1e-5 of expf here
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int key = 32 * t + 8 * (r / 4) + 4 * lh + (r % 4);
                const float val = key < T ? __fmul_rn(s[t][r], p.scale) : -INFINITY;
                s[t][r] = val;
                mx = fmaxf(mx, val);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        float sum = 0.0f;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float e = __builtin_amdgcn_exp2f(__fmul_rn(__fsub_rn(s[t][r], mx), 1.44269504088896340736f));
                s[t][r] = e;
                sum += e;
            }
        sum += __shfl_xor(sum, 32, 64);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int t = 0; t < NKT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[t][r] = __fmul_rn(s[t][r], inv);
    }

    // everybody is done with k: v takes its place
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int f = tid + i * 256;
        const int key = f / PARTS, part = f % PARTS;
        if (f < KEYS * PARTS) *reinterpret_cast<float4 *>(lds + key * LDV + part * 4) = vreg[i];
    }
    __syncthreads();
    if (!active) return;

    // out^T = v^T P^T: step (t, r) reduces over the keys the two lane halves hold in register r of tile t; groups of four
    // steps whose keys all lie past the last one are skipped (their probabilities are zero)
    f32x16 o[DT];
#pragma unroll
    for (int d = 0; d < DT; ++d)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[d][r] = 0.0f;
#pragma unroll
    for (int t = 0; t < NKT; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            if (32 * t + 8 * g >= T) continue;   // uniform
#pragma unroll
            for (int r = 4 * g; r < 4 * g + 4; ++r) {
                const int key = 32 * t + 8 * (r / 4) + 4 * lh + (r % 4);
#pragma unroll
                for (int d = 0; d < DT; ++d)
                    o[d] = __builtin_amdgcn_mfma_f32_32x32x2f32(lds[key * LDV + 32 * d + li], s[t][r], o[d], 0, 0, 0);
            }
        }

    if (query < T) {
        float *ob = p.o + b * p.os[0] + h * p.os[1] + (long long) query * p.os[2];
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<float4 *>(ob + 32 * d + 8 * g + 4 * lh) =
                    make_float4(o[d][4 * g], o[d][4 * g + 1], o[d][4 * g + 2], o[d][4 * g + 3]);
    }
}

template <int NKT, int HD>
static int attention_launch_one(const AttnParams &p, int batch, hipStream_t stream) {
    const dim3 grid((unsigned) ((p.tokens + 127) / 128), (unsigned) (batch * p.heads));
    hipLaunchKernelGGL((attention_f32_kernel<NKT, HD>), grid, dim3(256), 0, stream, p);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

template <int HD>
static int attention_launch_hd(const AttnParams &p, int batch, hipStream_t stream) {
    const int nkt = (p.tokens + 31) / 32;
    if (nkt <= 2) return attention_launch_one<2, HD>(p, batch, stream);
    if (nkt <= 4) return attention_launch_one<4, HD>(p, batch, stream);
    if (nkt <= 7) return attention_launch_one<7, HD>(p, batch, stream);
    return attention_launch_one<8, HD>(p, batch, stream);
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
    p.scale = d.scale;
    if (d.head_dim == 64) return attention_launch_hd<64>(p, d.batch, stream);
    return attention_launch_hd<32>(p, d.batch, stream);
}

}  // namespace onhip
