// Block-sparse flash-attention forward for llsa_l1 / llsa_l2.
//
// One wave owns one query block (16 queries).  All products run on the bf16 16x16x32 MFMA
// in the "transposed" orientation, keys on the M axis and queries on the N axis:
//     S^T (16 keys x 16 queries) = K_blk (16x64) . Q^T            A = R tile of K, B = R tile of Q
//     O^T (64 ch  x 16 queries) += V_blk^T (64x32 keys) . P^T     A = T tiles of V, B = P^T
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

#ifndef LLSA_FWD_NB
#define LLSA_FWD_NB 2          // 16-key blocks per pipeline step (2 or 4)
#endif

namespace llsa {

struct SoftmaxState {
    float m2;        // running max, in log2 units (score / sqrt(D) * log2 e)
    float lsum;      // this lane's share of the running sum, in units of the current weight
    f32x4 acc[4];    // O^T: channel 16*dt + 4*(l/16) + e of query l%16
};

// Operands of one step = NB 16-key blocks, as they sit in registers between load and use.
template <int NB>
struct KvRegs {
    bf16x8 k[NB][2];     // K rows (R tile): block j, channel half
    bf16x4 v[NB][4];     // V (T tile): block j, channel tile dt, keys 4*(l/16)..+3
};

// Where one step's blocks live: kb[j] is the R tile of key block j, vtb[j] the T tile of its values.
template <int NB>
struct StepDesc {
    const bf16* kb[NB];
    const bf16* vtb[NB];
    float wratio;        // weight(previous segment) / weight(this segment) on the first step of a segment
};

template <int NB>
__device__ __forceinline__ void load_step(KvRegs<NB>& t, const StepDesc<NB>& d, int lane) {
#pragma unroll
    for (int j = 0; j < NB; j++) {
        t.k[j][0] = ld16(d.kb[j] + lane * 8);
        t.k[j][1] = ld16(d.kb[j] + 512 + lane * 8);
    }
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++) t.v[j][dt] = ld8(d.vtb[j] + dt * 256 + lane * 4);
}

template <int NB>
__device__ __forceinline__ void compute_step(SoftmaxState& st, const bf16x8 bq[2], const KvRegs<NB>& t, float wratio) {
    f32x4 s[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        f32x4 z = {0.f, 0.f, 0.f, 0.f};
        z = mfma_bf16(t.k[j][0], bq[0], z);
        s[j] = mfma_bf16(t.k[j][1], bq[1], z);
    }
    float mx = s[0][0];
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) mx = fmaxf(mx, s[j][e]);
    mx = quad_max(mx);
    const float m2n = fmaxf(st.m2, mx * kScaleLog2e);
    const float alpha = exp2_fast(st.m2 - m2n) * wratio;
    float rs = 0.f;
    bf16x8 bp[NB / 2];
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float p = exp2_fast(fmaf(s[j][e], kScaleLog2e, -m2n));
            rs += p;
            bp[j >> 1][(j & 1) * 4 + e] = (bf16)p;
        }
    st.lsum = st.lsum * alpha + rs;
    st.m2 = m2n;
    if (__ballot(alpha != 1.f) != 0) {        // the running max moved (or a new segment starts) somewhere in the wave
#pragma unroll
        for (int dt = 0; dt < 4; dt++) st.acc[dt] *= alpha;
    }
#pragma unroll
    for (int c = 0; c < NB / 2; c++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
            st.acc[dt] = mfma_bf16(cat(t.v[2 * c][dt], t.v[2 * c + 1][dt]), bp[c], st.acc[dt]);
}

// One wave per query block; the KV list is walked in steps of NB blocks with the loads of
// step t+1 issued before the arithmetic of step t (two register buffers, ping-pong).
template <int NB>
__global__ __launch_bounds__(256) void attn_fwd_kernel(llsa_attn_fwd_args a) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int N1 = a.N / kBlk, N2 = N1 / kBlk;
    const int lid = xcd_logical_id();
    const int g = (lid % (int)gridDim.x) * 4 + wave;
    if (g >= N1) return;
    const int bh = lid / (int)gridDim.x, b = bh / a.H, h = bh % a.H;
    const int r = lane & 15, quad = lane >> 4;

    bf16x8 bq[2];
    {
        const bf16* qp = (const bf16*)a.qr + ((int64_t)bh * N1 + g) * kTile + lane * 8;
        bq[0] = ld16(qp);       // 1/sqrt(64) is a power of two: scaling q before the product (as the
        bq[1] = ld16(qp + 512); // reference does) equals scaling the fp32 scores, done in the exponent
    }
    SoftmaxState st;
    st.m2 = -INFINITY;
    st.lsum = 0.f;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) st.acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const bf16* kr = (const bf16*)a.kr + (int64_t)bh * N1 * kTile;
    const bf16* vt = (const bf16*)a.vt + (int64_t)bh * N1 * kTile;
    const bf16* pk = (const bf16*)a.pkr + (int64_t)bh * N2 * kTile;
    const bf16* pvt = (const bf16*)a.pvt + (int64_t)bh * N2 * kTile;
    const bf16* pk2 = (a.levels == 2) ? (const bf16*)a.pk2r + (int64_t)bh * (N2 / kBlk) * kTile : nullptr;
    const bf16* pv2t = (a.levels == 2) ? (const bf16*)a.pv2t + (int64_t)bh * (N2 / kBlk) * kTile : nullptr;
    const int* ip = a.idx + ((int64_t)bh * N1 + g) * a.T;
    const int* pip = (a.levels == 2) ? a.pidx + ((int64_t)bh * N2 + g / kBlk) * a.T2 : nullptr;

    // step t of the KV list: fine blocks, then (l2) the parent's level-1 pooled blocks, then
    // every block of the coarsest pooled level
    const int n_fine = a.T / NB;
    const int n_mid = (a.levels == 2) ? a.T2 / NB : 0;
    const int n_dense = ((a.levels == 2) ? N2 / kBlk : N1 / kBlk) / NB;
    const int n_steps = n_fine + n_mid + n_dense;
    const float w_last = (a.levels == 2) ? a.w2 : a.w1;
    auto describe = [&](int t, StepDesc<NB>& d) {
        if (t < n_fine) {
#pragma unroll
            for (int j = 0; j < NB; j++) {
                const int blk = clampi(ip[NB * t + j], 0, N1 - 1);
                d.kb[j] = kr + (int64_t)blk * kTile;
                d.vtb[j] = vt + (int64_t)blk * kTile;
            }
            d.wratio = 1.f;
        } else if (t < n_fine + n_mid) {
            const int u = t - n_fine;
#pragma unroll
            for (int j = 0; j < NB; j++) {
                const int blk = clampi(pip[NB * u + j], 0, N2 - 1);
                d.kb[j] = pk + (int64_t)blk * kTile;
                d.vtb[j] = pvt + (int64_t)blk * kTile;
            }
            d.wratio = (u == 0) ? 1.f / a.w1 : 1.f;
        } else {
            const int u = t - n_fine - n_mid;
            const bf16* kk = (a.levels == 2) ? pk2 : pk;
            const bf16* vv = (a.levels == 2) ? pv2t : pvt;
#pragma unroll
            for (int j = 0; j < NB; j++) {
                d.kb[j] = kk + (int64_t)(NB * u + j) * kTile;
                d.vtb[j] = vv + (int64_t)(NB * u + j) * kTile;
            }
            d.wratio = (u == 0) ? ((a.levels == 2) ? a.w1 / a.w2 : 1.f / a.w1) : 1.f;
        }
    };

    // The prefetch is unconditional (past the end it re-reads the last step) so that the loop
    // body is straight-line code: with the loads inside a branch the compiler has to drain the
    // memory queue (s_waitcnt vmcnt(0)) before every step and the overlap is lost.
    KvRegs<NB> ra, rb;
    StepDesc<NB> d;
    float wa, wb;
    describe(0, d);
    load_step(ra, d, lane);
    wa = d.wratio;
    for (int t = 0; t < n_steps; t += 2) {
        describe(min(t + 1, n_steps - 1), d);
        load_step(rb, d, lane);
        wb = d.wratio;
        compute_step(st, bq, ra, wa);
        if (t + 1 >= n_steps) break;
        describe(min(t + 2, n_steps - 1), d);
        load_step(ra, d, lane);
        wa = d.wratio;
        compute_step(st, bq, rb, wb);
    }

    const float L = quad_sum(st.lsum);
    const float inv = 1.f / L;
    bf16* op = (bf16*)a.o + b * a.sob + h * a.soh + (int64_t)(g * kBlk + r) * a.son + quad * 4;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) st8(op + dt * 16, cvt4(st.acc[dt] * inv));
    if (quad == 0) a.lse[(int64_t)bh * a.N + g * kBlk + r] = (st.m2 + __builtin_amdgcn_logf(L * w_last)) * kLn2;
}

}  // namespace llsa

using namespace llsa;

extern "C" int llsa_attn_fwd(const llsa_attn_fwd_args* a, void* stream) {
    LLSA_REQUIRE(a != nullptr, "attn_fwd: null args");
    LLSA_REQUIRE(a->levels == 1 || a->levels == 2, "attn_fwd: levels must be 1 or 2");
    LLSA_REQUIRE(a->B > 0 && a->H > 0 && a->N > 0, "attn_fwd: bad B/H/N");
    LLSA_REQUIRE(a->qr && a->kr && a->vt && a->pkr && a->pvt && a->idx && a->o && a->lse, "attn_fwd: null tensor");
    LLSA_REQUIRE(a->T >= 4 && a->T % 4 == 0 && a->T <= a->N / 16, "attn_fwd: topk=%d must be a multiple of 4 and <= N/16", a->T);
    LLSA_REQUIRE(a->w1 > 0.f, "attn_fwd: token_weight must be > 0");
    if (a->levels == 1) {
        LLSA_REQUIRE(a->N % 1024 == 0, "attn_fwd: llsa_l1 needs N %% 1024 == 0 (N=%d): the coarse loop runs over 64-token tiles of N/16 pooled tokens", a->N);
    } else {
        LLSA_REQUIRE(a->N % 16384 == 0, "attn_fwd: llsa_l2 needs N %% 16384 == 0 (N=%d): the level-2 loop runs over 64-token tiles of N/256 pooled tokens", a->N);
        LLSA_REQUIRE(a->pk2r && a->pv2t && a->pidx, "attn_fwd: level-2 tensors missing");
        LLSA_REQUIRE(a->T2 >= 4 && a->T2 % 4 == 0 && a->T2 <= a->N / 256, "attn_fwd: topk2=%d must be a multiple of 4 and <= N/256", a->T2);
        LLSA_REQUIRE(a->w2 > 0.f, "attn_fwd: token_weight_2 must be > 0");
    }
    LLSA_REQUIRE(aligned16(a->qr) && aligned16(a->kr) && aligned16(a->vt) && aligned16(a->pkr) && aligned16(a->pvt) &&
                     aligned16(a->pk2r) && aligned16(a->pv2t) && aligned16(a->o),
                 "attn_fwd: tensors must be 16-byte aligned");
    LLSA_REQUIRE((a->sob % 4 == 0) && (a->soh % 4 == 0) && (a->son % 4 == 0), "attn_fwd: rows of o must be 8-byte aligned");
    const int N1 = a->N / 16;
    hipLaunchKernelGGL(HIP_KERNEL_NAME(attn_fwd_kernel<LLSA_FWD_NB>), dim3((N1 + 3) / 4, a->B * a->H), dim3(256), 0,
                       (hipStream_t)stream, *a);
    return launch_status("attn_fwd");
}
