// Attention with 16-bit operands (bf16 / fp16 q, k, v and result in memory, fp32 scores and Softmax): the 16-bit storage
// form of attention.hip, same chain of reference operators (device/x86/MatMul/mat_mul.c:10-102, device/x86/Softmax/
// softmax.c:26-59, Transposes folded into strides), same trick: a wavefront computes the TRANSPOSED scores S^T = k q^T
// with v_mfma_f32_32x32x16_{bf16,f16}, so a lane owns one query and, per 32-key tile, the 16 keys 8 (r / 4) + 4 (lane / 32)
// + r % 4, the Softmax is a reduction inside the lane, and the probabilities feed the second product out^T = v^T P^T from
// the registers they are in.  An MFMA step of the second product takes 8 reduction indices per lane half: registers
// 8 g .. 8 g + 7 of a tile, i.e. the keys 32 t + 16 g + 8 (j / 4) + 4 (lane / 32) + j % 4, rounded to the 16-bit type and
// packed; the A operand for them is two 8-byte reads of v^T[channel lane % 32][key], which is why v is transposed on its
// way into LDS (k is copied as it is).  The probabilities are rounded to the operand type before the second product: that
// is what 16-bit operands mean for a MatMul; everything before it (scores, maximum, exponentials, sum, normalisation) is
// fp32.  Head dimension 64, at most 256 tokens.
#include "igemm_kernel.hpp"

namespace onhip {

struct AttnH16Params {
    const unsigned short *q, *k, *v;
    unsigned short *o;
    long long qs[3], ks[3], vs[3], os[3];   // element strides of (batch, head, token); the head dimension is contiguous
    int heads, tokens;
    float scale;
};

template <int DT, int NKT>
__global__ __launch_bounds__(256, 2) void attention_h16_kernel(const AttnH16Params p) {
    constexpr int HD = 64, KEYS = NKT * 32;
    constexpr int LDK = HD + 8;       // 16-bit elements per key row of k (144 bytes: 16-byte reads of neighbouring rows spread over the banks)
    constexpr int LDVT = KEYS + 8;    // 16-bit elements per channel row of v^T
    __shared__ __attribute__((aligned(16))) unsigned short Ks[KEYS * LDK];
    __shared__ __attribute__((aligned(16))) unsigned short Vt[HD * LDVT];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 31, lh = lane >> 5;
    const int bh = blockIdx.y, b = bh / p.heads, h = bh - b * p.heads;
    const int T = p.tokens;
    const unsigned short *kb = p.k + b * p.ks[0] + h * p.ks[1];
    const unsigned short *vb = p.v + b * p.vs[0] + h * p.vs[1];

    // k rows as they are, v transposed; rows / columns past the last key as zeros.  All loads first.
    constexpr int PARTS = HD / 8, NV = (KEYS * PARTS + 255) / 256;
    uint4 kq[NV], vq[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int f = tid + i * 256;
        const int key = f / PARTS, part = f % PARTS;
        kq[i] = vq[i] = make_uint4(0u, 0u, 0u, 0u);
        if (key < T) {
            kq[i] = *reinterpret_cast<const uint4 *>(kb + key * p.ks[2] + part * 8);
            vq[i] = *reinterpret_cast<const uint4 *>(vb + key * p.vs[2] + part * 8);
        }
    }
    // this lane's query row: the channels 16 s + 8 (lane / 32) .. + 7 of MFMA step s
    const int q0 = (blockIdx.x * 4 + wave) * 32;
    const int query = q0 + li;
    uint4 qf[HD / 16];
    {
        const unsigned short *qb = p.q + b * p.qs[0] + h * p.qs[1] + (long long) query * p.qs[2];
#pragma unroll
        for (int s = 0; s < HD / 16; ++s)
            qf[s] = query < T ? *reinterpret_cast<const uint4 *>(qb + 16 * s + 8 * lh) : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int f = tid + i * 256;
        const int key = f / PARTS, part = f % PARTS;
        if (f < KEYS * PARTS) {
            *reinterpret_cast<uint4 *>(Ks + key * LDK + part * 8) = kq[i];
            const unsigned w[4] = {vq[i].x, vq[i].y, vq[i].z, vq[i].w};
#pragma unroll
            for (int e = 0; e < 8; ++e) Vt[(part * 8 + e) * LDVT + key] = (unsigned short) (w[e / 2] >> (16 * (e & 1)));
        }
    }
    __syncthreads();
    if (q0 >= T) return;   // a wavefront without queries (uniform); nothing below synchronises

    auto mfma = [](const uint4 &a, const uint4 &bq, f32x16 c) __attribute__((always_inline)) {
        if constexpr (DT == DT_BF16)
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, bq), c, 0, 0, 0);
        else
            return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, bq), c, 0, 0, 0);
    };

    // S^T = k q^T
    f32x16 s[NKT];
#pragma unroll
    for (int t = 0; t < NKT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[t][r] = 0.0f;
#pragma unroll
    for (int st = 0; st < HD / 16; ++st) {
        uint4 kf[NKT];
#pragma unroll
        for (int t = 0; t < NKT; ++t) kf[t] = *reinterpret_cast<const uint4 *>(Ks + (32 * t + li) * LDK + 16 * st + 8 * lh);
#pragma unroll
        for (int t = 0; t < NKT; ++t) s[t] = mfma(kf[t], qf[st], s[t]);
    }

    // Softmax over the keys in fp32 (softmax.c:26-59); keys past the last count as minus infinity
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

    // out^T = v^T P^T, the probabilities normalised, rounded and packed eight at a time
    f32x16 o[2];
#pragma unroll
    for (int d = 0; d < 2; ++d)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[d][r] = 0.0f;
#pragma unroll
    for (int t = 0; t < NKT; ++t)
#pragma unroll
        for (int g = 0; g < 2; ++g) {
            if (32 * t + 16 * g >= T) continue;   // uniform: all of these keys lie past the last one
            uint4 pq;
            pq.x = pack_h16<DT>(__fmul_rn(s[t][8 * g + 0], inv), __fmul_rn(s[t][8 * g + 1], inv));
            pq.y = pack_h16<DT>(__fmul_rn(s[t][8 * g + 2], inv), __fmul_rn(s[t][8 * g + 3], inv));
            pq.z = pack_h16<DT>(__fmul_rn(s[t][8 * g + 4], inv), __fmul_rn(s[t][8 * g + 5], inv));
            pq.w = pack_h16<DT>(__fmul_rn(s[t][8 * g + 6], inv), __fmul_rn(s[t][8 * g + 7], inv));
            const int key0 = 32 * t + 16 * g + 4 * lh;   // slots 0..3: key0 .. key0 + 3, slots 4..7: key0 + 8 .. key0 + 11
#pragma unroll
            for (int d = 0; d < 2; ++d) {
                const unsigned short *vr = Vt + (32 * d + li) * LDVT + key0;
                const uint2 lo = *reinterpret_cast<const uint2 *>(vr), hi = *reinterpret_cast<const uint2 *>(vr + 8);
                o[d] = mfma(make_uint4(lo.x, lo.y, hi.x, hi.y), pq, o[d]);
            }
        }

    if (query < T) {
        unsigned short *ob = p.o + b * p.os[0] + h * p.os[1] + (long long) query * p.os[2];
#pragma unroll
        for (int d = 0; d < 2; ++d)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<uint2 *>(ob + 32 * d + 8 * g + 4 * lh) =
                    make_uint2(pack_h16<DT>(o[d][4 * g], o[d][4 * g + 1]), pack_h16<DT>(o[d][4 * g + 2], o[d][4 * g + 3]));
    }
}

template <int DT>
static int attention_h16_launch_dt(const AttnH16Params &p, int batch, hipStream_t stream) {
    const dim3 grid((unsigned) ((p.tokens + 127) / 128), (unsigned) (batch * p.heads));
    const int nkt = (p.tokens + 31) / 32;
    if (nkt <= 2) hipLaunchKernelGGL((attention_h16_kernel<DT, 2>), grid, dim3(256), 0, stream, p);
    else if (nkt <= 4) hipLaunchKernelGGL((attention_h16_kernel<DT, 4>), grid, dim3(256), 0, stream, p);
    else if (nkt <= 7) hipLaunchKernelGGL((attention_h16_kernel<DT, 7>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((attention_h16_kernel<DT, 8>), grid, dim3(256), 0, stream, p);
    ONHIP_CHECK_HIP(hipGetLastError());
    return ONHIP_OK;
}

int attention_h16_launch(int dt, const onhip_attention_desc_t &d, const void *q, const void *k, const void *v, void *out,
                         hipStream_t stream) {
    AttnH16Params p;
    p.q = reinterpret_cast<const unsigned short *>(q);
    p.k = reinterpret_cast<const unsigned short *>(k);
    p.v = reinterpret_cast<const unsigned short *>(v);
    p.o = reinterpret_cast<unsigned short *>(out);
    for (int i = 0; i < 3; ++i) {
        p.qs[i] = d.q_strides[i]; p.ks[i] = d.k_strides[i]; p.vs[i] = d.v_strides[i]; p.os[i] = d.out_strides[i];
    }
    p.heads = d.heads;
    p.tokens = d.tokens;
    p.scale = d.scale;
    return dt == DT_BF16 ? attention_h16_launch_dt<DT_BF16>(p, d.batch, stream) : attention_h16_launch_dt<DT_F16>(p, d.batch, stream);
}

}  // namespace onhip
