// Block-sparse flash-attention forward for llsa_l1 / llsa_l2.
//
// One wave owns one query block (16 queries).  All products run on the bf16 16x16x32 MFMA
// in the "transposed" orientation, keys on the M axis and queries on the N axis:
//     S^T (16 keys x 16 queries) = K_blk (16x64) . Q^T            A = K rows, B = Q rows
//     O^T (64 ch  x 16 queries) += V_blk^T (64x32 keys) . P^T     A = block-transposed V, B = P^T
// With this orientation lane l holds, for query l%16, the scores of keys 4*(l/16)..+3 of a
// tile -- which is exactly the B-operand layout of the second product -- and the O^T
// accumulator of lane l belongs to the same query, so the soft-max statistics (running
// max, running sum, rescale factor) never leave the lane that needs them; a row reduction
// is two cross-lane steps (lanes l, l^16, l^32, l^48).
//
// KV order per query block: T selected 16-token blocks of K/V, then (l2) the 16*T2 level-1
// pooled tokens inside the parent's selected coarse blocks, then every token of the
// coarsest pooled level.  Pooled segments count with weight w1 / w2: the accumulator and
// the running sum are kept in units of the current segment's weight, converted once at
// each segment boundary.
#include "llsa_device.h"
#include "llsa_host.h"
#include "../../include/llsa_hip.h"

namespace llsa {

struct SoftmaxState {
    float m2;        // running max, in log2 units (score / sqrt(D) * log2 e)
    float lsum;      // this lane's share of the running sum, in units of the current weight
    f32x4 acc[4];    // O^T: channel 16*dt + 4*(l/16) + e of query l%16
};

// One 64-key tile = four 16-key blocks.  kb[j] points at row 0 of block j (row stride ks
// elements), vtb[j] at the block-transposed values of block j.
__device__ __forceinline__ void fwd_tile(SoftmaxState& st, const bf16x8 bq[2], const bf16* const kb[4], int64_t ks,
                                         const bf16* const vtb[4], float wratio, int lane) {
    const int r = lane & 15, quad = lane >> 4;
    f32x4 s[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const bf16* p = kb[j] + r * ks + quad * 8;
        f32x4 z = {0.f, 0.f, 0.f, 0.f};
        z = mfma_bf16(ld16(p), bq[0], z);
        s[j] = mfma_bf16(ld16(p + 32), bq[1], z);
    }
    float mx = s[0][0];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) mx = fmaxf(mx, s[j][e]);
    mx = quad_max(mx);
    const float m2n = fmaxf(st.m2, mx * kScaleLog2e);
    const float alpha = exp2_fast(st.m2 - m2n) * wratio;
    float rs = 0.f;
    bf16x8 bp[2];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float p = exp2_fast(fmaf(s[j][e], kScaleLog2e, -m2n));
            rs += p;
            bp[j >> 1][(j & 1) * 4 + e] = (bf16)p;
        }
    st.lsum = st.lsum * alpha + rs;
    st.m2 = m2n;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) st.acc[dt] *= alpha;
#pragma unroll
    for (int c = 0; c < 2; c++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
            const int off = (dt * 16 + r) * kBlk + quad * 4;
            st.acc[dt] = mfma_bf16(cat(ld8(vtb[2 * c] + off), ld8(vtb[2 * c + 1] + off)), bp[c], st.acc[dt]);
        }
}

__global__ __launch_bounds__(256) void attn_fwd_kernel(llsa_attn_fwd_args a) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int N1 = a.N / kBlk, N2 = N1 / kBlk;
    const int g = blockIdx.x * 4 + wave;
    if (g >= N1) return;
    const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
    const int r = lane & 15, quad = lane >> 4;

    bf16x8 bq[2];
    {
        const bf16* qp = (const bf16*)a.q + b * a.sqb + h * a.sqh + (int64_t)(g * kBlk + r) * a.sqn + quad * 8;
        bq[0] = ld16(qp);      // 1/sqrt(64) is a power of two: scaling q before the product (as the
        bq[1] = ld16(qp + 32); // reference does) equals scaling the fp32 scores, done in the exponent
    }
    SoftmaxState st;
    st.m2 = -INFINITY;
    st.lsum = 0.f;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) st.acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const bf16* kbase = (const bf16*)a.k + b * a.skb + h * a.skh;
    const bf16* vt = (const bf16*)a.vt + (int64_t)bh * N1 * (kD * kBlk);
    const bf16* pk = (const bf16*)a.pk + (int64_t)bh * N1 * kD;
    const bf16* pvt = (const bf16*)a.pvt + (int64_t)bh * N2 * (kD * kBlk);
    const bf16* kb[4];
    const bf16* vtb[4];

    const int* ip = a.idx + ((int64_t)bh * N1 + g) * a.T;
    for (int t = 0; t < a.T / 4; t++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int blk = clampi(ip[4 * t + j], 0, N1 - 1);
            kb[j] = kbase + (int64_t)blk * kBlk * a.skn;
            vtb[j] = vt + (int64_t)blk * (kD * kBlk);
        }
        fwd_tile(st, bq, kb, a.skn, vtb, 1.f, lane);
    }
    float wcur;
    if (a.levels == 2) {
        const int* pip = a.pidx + ((int64_t)bh * N2 + g / kBlk) * a.T2;
        for (int t = 0; t < a.T2 / 4; t++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int blk = clampi(pip[4 * t + j], 0, N2 - 1);
                kb[j] = pk + (int64_t)blk * kBlk * kD;
                vtb[j] = pvt + (int64_t)blk * (kD * kBlk);
            }
            fwd_tile(st, bq, kb, kD, vtb, t == 0 ? 1.f / a.w1 : 1.f, lane);
        }
        const bf16* pk2 = (const bf16*)a.pk2 + (int64_t)bh * N2 * kD;
        const bf16* pv2t = (const bf16*)a.pv2t + (int64_t)bh * (N2 / kBlk) * (kD * kBlk);
        for (int t = 0; t < N2 / 64; t++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                kb[j] = pk2 + (int64_t)(4 * t + j) * kBlk * kD;
                vtb[j] = pv2t + (int64_t)(4 * t + j) * (kD * kBlk);
            }
            fwd_tile(st, bq, kb, kD, vtb, t == 0 ? a.w1 / a.w2 : 1.f, lane);
        }
        wcur = a.w2;
    } else {
        for (int t = 0; t < N1 / 64; t++) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                kb[j] = pk + (int64_t)(4 * t + j) * kBlk * kD;
                vtb[j] = pvt + (int64_t)(4 * t + j) * (kD * kBlk);
            }
            fwd_tile(st, bq, kb, kD, vtb, t == 0 ? 1.f / a.w1 : 1.f, lane);
        }
        wcur = a.w1;
    }

    const float L = quad_sum(st.lsum);
    const float inv = 1.f / L;
    bf16* op = (bf16*)a.o + b * a.sob + h * a.soh + (int64_t)(g * kBlk + r) * a.son + quad * 4;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) st8(op + dt * 16, cvt4(st.acc[dt] * inv));
    if (quad == 0) a.lse[(int64_t)bh * a.N + g * kBlk + r] = (st.m2 + __builtin_amdgcn_logf(L * wcur)) * kLn2;
}

}  // namespace llsa

using namespace llsa;

extern "C" int llsa_attn_fwd(const llsa_attn_fwd_args* a, void* stream) {
    LLSA_REQUIRE(a != nullptr, "attn_fwd: null args");
    LLSA_REQUIRE(a->levels == 1 || a->levels == 2, "attn_fwd: levels must be 1 or 2");
    LLSA_REQUIRE(a->B > 0 && a->H > 0 && a->N > 0, "attn_fwd: bad B/H/N");
    LLSA_REQUIRE(a->q && a->k && a->vt && a->pk && a->pvt && a->idx && a->o && a->lse, "attn_fwd: null tensor");
    LLSA_REQUIRE(a->T >= 4 && a->T % 4 == 0 && a->T <= a->N / 16, "attn_fwd: topk=%d must be a multiple of 4 and <= N/16", a->T);
    LLSA_REQUIRE(a->w1 > 0.f, "attn_fwd: token_weight must be > 0");
    if (a->levels == 1) {
        LLSA_REQUIRE(a->N % 1024 == 0, "attn_fwd: llsa_l1 needs N %% 1024 == 0 (N=%d): the coarse loop runs over 64-token tiles of N/16 pooled tokens", a->N);
    } else {
        LLSA_REQUIRE(a->N % 16384 == 0, "attn_fwd: llsa_l2 needs N %% 16384 == 0 (N=%d): the level-2 loop runs over 64-token tiles of N/256 pooled tokens", a->N);
        LLSA_REQUIRE(a->pk2 && a->pv2t && a->pidx, "attn_fwd: level-2 tensors missing");
        LLSA_REQUIRE(a->T2 >= 4 && a->T2 % 4 == 0 && a->T2 <= a->N / 256, "attn_fwd: topk2=%d must be a multiple of 4 and <= N/256", a->T2);
        LLSA_REQUIRE(a->w2 > 0.f, "attn_fwd: token_weight_2 must be > 0");
    }
    LLSA_REQUIRE(aligned16(a->q) && aligned16(a->k) && aligned16(a->vt) && aligned16(a->pk) && aligned16(a->pvt) &&
                     aligned16(a->pk2) && aligned16(a->pv2t) && aligned16(a->o),
                 "attn_fwd: tensors must be 16-byte aligned");
    LLSA_REQUIRE(stride_ok(a->sqb) && stride_ok(a->sqh) && stride_ok(a->sqn) && stride_ok(a->skb) && stride_ok(a->skh) &&
                     stride_ok(a->skn) && (a->sob % 4 == 0) && (a->soh % 4 == 0) && (a->son % 4 == 0),
                 "attn_fwd: row strides must keep rows 16-byte aligned");
    const int N1 = a->N / 16;
    hipLaunchKernelGGL(attn_fwd_kernel, dim3((N1 + 3) / 4, a->B * a->H), dim3(256), 0, (hipStream_t)stream, *a);
    return launch_status("attn_fwd");
}
