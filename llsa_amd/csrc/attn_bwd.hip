// Backward of the block-sparse attention: delta pre-pass, dQ per query block, and the
// K-side gradients (dK/dV of the fine tokens through the transposed index, the sparse
// level-1 pooled gradients of llsa_l2, and the dense coarsest pooled gradients).
//
// MFMA orientations (bf16 16x16x32, see llsa_device.h for the register layout):
//   dQ pass, per key block (keys on M, queries on N, like the forward):
//       S^T  = K . Q^T          dP^T = V . dO^T          dS^T = P^T o (dP^T - delta)
//       dQ^T (64 ch x 16 q) += K_blk^T (64 x 32 keys) . dS^T      A = block-transposed K
//   K-side pass, per key block and per pair of query blocks (queries on M, keys on N):
//       S    = Q . K^T          dP   = dO . V^T          dS   = P o (dP - delta)
//       dV^T (64 ch x 16 keys) += dO_blk^T (64 x 32 q) . P        A = block-transposed dO
//       dK^T (64 ch x 16 keys) += Q_blk^T  (64 x 32 q) . dS       A = block-transposed Q
// In both passes the score tile leaves the MFMA in exactly the operand layout the next
// product needs, so P and dS go from registers to registers.
#include "llsa_device.h"
#include "llsa_host.h"
#include "../../include/llsa_hip.h"

namespace llsa {

// ---------------------------------------------------------------------------------------
// dQ: one wave per query block, four consecutive query blocks per workgroup, key blocks taken
// two at a time (32 keys = one MFMA K step).
//
// K and V always reach the MFMA from R tiles.  K is needed twice: as the A operand of S^T (a plain
// 16-byte read per lane) and, read back with the transposing LDS load, as the A operand of
// dQ^T += K^T.dS^T -- so K goes through LDS in any case, copied there straight from global memory.
//  * pooled blocks (level-1 pooled tokens of the parent's coarse blocks, the coarsest level) are
//    the same for the four query blocks of the workgroup: one copy per workgroup, kGroup blocks
//    of K and V at a time, two buffers;
//  * fine blocks are private: afterwards each wave re-uses a quarter of the same LDS as two slots
//    for the K tiles of a pair (the copy of pair t+1 in flight during pair t), V stays in registers.
// ---------------------------------------------------------------------------------------
struct PairR {
    bf16x8 k[2][2], v[2][2];       // block j, channel half
};
struct PairT {
    bf16x4 t[2][4];                // block j, channel tile dt
};

__device__ __forceinline__ void read_k_r(PairR& o, const bf16* k0, const bf16* k1, int lane) {
    o.k[0][0] = lds_ld16(k0 + lane * 8);
    o.k[0][1] = lds_ld16(k0 + 512 + lane * 8);
    o.k[1][0] = lds_ld16(k1 + lane * 8);
    o.k[1][1] = lds_ld16(k1 + 512 + lane * 8);
}
__device__ __forceinline__ void read_v_r(PairR& o, const bf16* v0, const bf16* v1, int lane) {
    o.v[0][0] = lds_ld16(v0 + lane * 8);
    o.v[0][1] = lds_ld16(v0 + 512 + lane * 8);
    o.v[1][0] = lds_ld16(v1 + lane * 8);
    o.v[1][1] = lds_ld16(v1 + 512 + lane * 8);
}
__device__ __forceinline__ void read_k_t(PairT& o, const bf16* k0, const bf16* k1, int lane) {
#pragma unroll
    for (int dt = 0; dt < 4; dt++) {
        o.t[0][dt] = lds_t_operand(k0, dt, lane);
        o.t[1][dt] = lds_t_operand(k1, dt, lane);
    }
}
// dS^T of a pair of key blocks, as the B operand of the dQ product
// (lse2w: the query's log-sum-exp minus log2 of the segment's weight, log2 units: the weight rides in the exponent)
__device__ __forceinline__ bf16x8 dq_scores(const PairR& p, const bf16x8 bq[2], const bf16x8 bdo[2], float lse2w,
                                            float delta) {
    bf16x8 bds;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        f32x4 s = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
        s = mfma_bf16(p.k[j][0], bq[0], s);
        s = mfma_bf16(p.k[j][1], bq[1], s);
        dp = mfma_bf16(p.v[j][0], bdo[0], dp);
        dp = mfma_bf16(p.v[j][1], bdo[1], dp);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float pe = exp2_fast(fmaf(s[e], kScaleLog2e, -lse2w));
            bds[j * 4 + e] = (bf16)(pe * (dp[e] - delta));
        }
    }
    return bds;
}
__device__ __forceinline__ void dq_accum(f32x4 dq[4], const PairT& p, bf16x8 bds) {
#pragma unroll
    for (int dt = 0; dt < 4; dt++) dq[dt] = mfma_bf16(cat(p.t[0][dt], p.t[1][dt]), bds, dq[dt]);
}

// What a wave keeps per query block
struct DqSide {
    bf16x8 bq[2], bdo[2];          // R operands of q and dO
    float lse2, dl;                // log-sum-exp (log2 units) and delta of query l%16
    f32x4 dq[4];                   // dQ^T: channel 16*dt + 4*(l/16) + e of query l%16
};

// dO comes straight from the caller's tensor, already in the register layout of an R operand
// (lane l: row l%16, channels 8*(l/16)..+7 and 32 + 8*(l/16)..+7).  The wave also does the
// pre-pass the K-side kernels need: delta = rowsum(O * dO) in fp32 (the reference sums in the
// tensor dtype, sparse_attention_res_1.py:153-177) and dO as an R tile.
__device__ __forceinline__ void dq_begin(DqSide& sd, const llsa_attn_bwd_args& a, float* __restrict__ delta, bf16* __restrict__ dor,
                                         int bh, int b, int h, int g, int lane) {
    const int N1 = a.N / kBlk, r = lane & 15, quad = lane >> 4, tok = g * kBlk + r;
    const bf16* qp = (const bf16*)a.qr + ((int64_t)bh * N1 + g) * kTile + lane * 8;
    sd.bq[0] = ld16(qp);
    sd.bq[1] = ld16(qp + 512);
    const bf16* gp = (const bf16*)a.dout + b * a.sdob + h * a.sdoh + (int64_t)tok * a.sdon + quad * 8;
    const bf16* op = (const bf16*)a.o + b * a.sob + h * a.soh + (int64_t)tok * a.son + quad * 8;
    sd.bdo[0] = ld16(gp);
    sd.bdo[1] = ld16(gp + 32);
    const bf16x8 o0 = ld16(op), o1 = ld16(op + 32);
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) acc += (float)o0[e] * (float)sd.bdo[0][e];
#pragma unroll
    for (int e = 0; e < 8; e++) acc += (float)o1[e] * (float)sd.bdo[1][e];
    sd.dl = quad_sum(acc);
    bf16* tile = dor + ((int64_t)bh * N1 + g) * kTile + lane * 8;
    st16(tile, sd.bdo[0]);
    st16(tile + 512, sd.bdo[1]);
    if (quad == 0) delta[(int64_t)bh * a.N + tok] = sd.dl;
    sd.lse2 = a.lse[(int64_t)bh * a.N + tok] * kLog2e;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) sd.dq[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
}
__device__ __forceinline__ void dq_end(const DqSide& sd, const llsa_attn_bwd_args& a, int b, int h, int g, int lane) {
    const int r = lane & 15, quad = lane >> 4, tok = g * kBlk + r;
    bf16* op = (bf16*)a.dq + b * a.sdqb + h * a.sdqh + (int64_t)tok * a.sdqn + quad * 4;
    const bf16* fq = a.freq_dq ? (const bf16*)a.freq_dq + (int64_t)tok * kD + quad * 4 : nullptr;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) {
        bf16x4 o = cvt4(sd.dq[dt] * kScale);
        if (fq != nullptr) o = rope_bwd4(o, ld8(fq + dt * 16));   // rotate the gradient back
        st8(op + dt * 16, o);
    }
}
__device__ __forceinline__ void dq_pair_of_blocks(DqSide& sd, const PairR& r, const PairT& t, float log2w) {
    dq_accum(sd.dq, t, dq_scores(r, sd.bq, sd.bdo, sd.lse2 - log2w, sd.dl));
}

__global__ __launch_bounds__(256) void attn_dq_kernel(llsa_attn_bwd_args a, float* __restrict__ delta,
                                                      bf16* __restrict__ dor) {
    __shared__ __align__(16) bf16 sh[2][kGroup][2 * kTile];   // per block: R tile of K, R tile of V
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int N1 = a.N / kBlk;
    const int lid = xcd_logical_id();
    const int g = (lid % (int)gridDim.x) * 4 + wave;          // < N1: the host checks N1 % 4 == 0
    const int bh = lid / (int)gridDim.x, b = bh / a.H, h = bh % a.H;

    const bf16* kr = (const bf16*)a.kr + (int64_t)bh * N1 * kTile;
    const bf16* vr = (const bf16*)a.vr + (int64_t)bh * N1 * kTile;
    const int* ip = a.idx + ((int64_t)bh * N1 + g) * a.T;

    // shared list: the selected blocks of every pooled level below the coarsest, then every block of the coarsest
    SharedList sl = shared_list(a.lvl, a.levels, a.N, bh, g, lane);
    const int n_groups = sl.n_blocks / kGroup;
    bf16* const sh0 = &sh[0][0][0];
    auto issue_group = [&](int grp) __attribute__((always_inline)) {   // this wave brings in block kGroup*grp + wave
        const SharedBlock sb = shared_block(sl, a.lvl, a.levels, a.N, bh, kGroup * grp + wave);
        const bf16* kb = (const bf16*)a.lvl[sb.level].kr + sb.tile;
        const bf16* vb = (const bf16*)a.lvl[sb.level].vr + sb.tile;
        bf16* dst = sh0 + ((grp & 1) * kGroup + wave) * (2 * kTile);
        copy16_global_to_lds(kb + lane * 8, dst);
        copy16_global_to_lds(kb + 512 + lane * 8, dst + 512);
        copy16_global_to_lds(vb + lane * 8, dst + kTile);
        copy16_global_to_lds(vb + 512 + lane * 8, dst + kTile + 512);
    };
    issue_group(0);
    int mine = (lane < min(kWave, a.T)) ? ip[lane] : 0;       // first 64 fine indices, entry i in lane i

    DqSide sd;
    dq_begin(sd, a, delta, dor, bh, b, h, g, lane);

    // ---- pooled blocks out of the shared copy.  The barrier at the top of round grp says: every
    // wave's part of group grp has landed, and every wave is done reading the other buffer.  All
    // LDS reads of a round come before the next fetch is issued (the compiler makes an LDS read
    // wait for every copy into LDS issued before it).
    for (int grp = 0; grp < n_groups; grp++) {
        wait_vm0();
        __syncthreads();
        const float w = __builtin_amdgcn_logf(a.lvl[shared_level(a.lvl, a.levels, kGroup * grp)].w);   // log2
        const bf16* blk = sh0 + (grp & 1) * kGroup * (2 * kTile);
        PairR r0;
        PairT t0;
        read_k_r(r0, blk, blk + 2 * kTile, lane);
        read_v_r(r0, blk + kTile, blk + 3 * kTile, lane);
        read_k_t(t0, blk, blk + 2 * kTile, lane);
        dq_pair_of_blocks(sd, r0, t0, w);
        read_k_r(r0, blk + 4 * kTile, blk + 6 * kTile, lane);
        read_v_r(r0, blk + 5 * kTile, blk + 7 * kTile, lane);
        read_k_t(t0, blk + 4 * kTile, blk + 6 * kTile, lane);
        if (grp + 1 < n_groups) issue_group(grp + 1);
        dq_pair_of_blocks(sd, r0, t0, w);
    }
    __syncthreads();                                          // the shared copy is dead: its LDS becomes private slots

    // ---- fine blocks: K of pair t+1 is copied into the wave's other slot and V of pair t+1 loaded
    // into registers while pair t is worked on.  Nothing may be in flight when the wave ends (a copy
    // landing in LDS that already belongs to another workgroup), so the last pair fetches nothing.
    bf16* const priv = sh0 + wave * (4 * kTile);              // two slots of two K tiles
    for (int c0 = 0; c0 < a.T; c0 += kWave) {
        const int cn = min(kWave, a.T - c0);
        if (c0 > 0) mine = (lane < cn) ? ip[c0 + lane] : 0;
        const int n_pairs = cn / 2;
        PairR ra, rb;
        auto fetch = [=](int t, PairR& dst) __attribute__((always_inline)) {
            bf16* slot = priv + (t & 1) * (2 * kTile);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int blk = clampi(__builtin_amdgcn_readlane(mine, 2 * t + j), 0, N1 - 1);
                const bf16* kb = kr + (int64_t)blk * kTile;
                const bf16* vb = vr + (int64_t)blk * kTile;
                copy16_global_to_lds(kb + lane * 8, slot + j * kTile);
                copy16_global_to_lds(kb + 512 + lane * 8, slot + j * kTile + 512);
                dst.v[j][0] = ld16(vb + lane * 8);
                dst.v[j][1] = ld16(vb + 512 + lane * 8);
            }
        };
        auto work = [&](int t, PairR& cur, PairR& nxt) __attribute__((always_inline)) {
            wait_vm0();
            const bf16* slot = priv + (t & 1) * (2 * kTile);
            PairT tt;
            read_k_r(cur, slot, slot + kTile, lane);
            read_k_t(tt, slot, slot + kTile, lane);
            if (t + 1 < n_pairs) fetch(t + 1, nxt);
            dq_pair_of_blocks(sd, cur, tt, 0.f);
        };
        fetch(0, ra);
        for (int t = 0; t < n_pairs; t += 2) {                // n_pairs is even (T % 4 == 0)
            work(t, ra, rb);
            work(t + 1, rb, ra);
        }
    }
    dq_end(sd, a, b, h, g, lane);
}

// Two sibling query blocks per wave (topk <= kPairMaxTopk): the pooled blocks and the fine blocks both rows
// selected are read once -- from memory and, what weighs more here, from LDS, where every key block is read
// three times (K rows, V rows, K transposed) -- and multiplied twice.  See pair_order for the walk.
__global__ __launch_bounds__(256, 3) void attn_dq_pair_kernel(llsa_attn_bwd_args a, float* __restrict__ delta,
                                                              bf16* __restrict__ dor) {
    __shared__ __align__(16) bf16 sh[2][kGroup][2 * kTile];
    __shared__ int order[4][kWave];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int N1 = a.N / kBlk, T = a.T;
    const int lid = xcd_logical_id();
    const int g = (lid % (int)gridDim.x) * 8 + 2 * wave;      // query blocks g and g + 1 (the host checks N1 % 8 == 0)
    const int bh = lid / (int)gridDim.x, b = bh / a.H, h = bh % a.H;

    const bf16* kr = (const bf16*)a.kr + (int64_t)bh * N1 * kTile;
    const bf16* vr = (const bf16*)a.vr + (int64_t)bh * N1 * kTile;
    const int* ip = a.idx + ((int64_t)bh * N1 + g) * T;

    SharedList sl = shared_list(a.lvl, a.levels, a.N, bh, g, lane);
    const int n_groups = sl.n_blocks / kGroup;
    bf16* const sh0 = &sh[0][0][0];
    auto issue_group = [&](int grp) __attribute__((always_inline)) {
        const SharedBlock sb = shared_block(sl, a.lvl, a.levels, a.N, bh, kGroup * grp + wave);
        const bf16* kb = (const bf16*)a.lvl[sb.level].kr + sb.tile;
        const bf16* vb = (const bf16*)a.lvl[sb.level].vr + sb.tile;
        bf16* dst = sh0 + ((grp & 1) * kGroup + wave) * (2 * kTile);
        copy16_global_to_lds(kb + lane * 8, dst);
        copy16_global_to_lds(kb + 512 + lane * 8, dst + 512);
        copy16_global_to_lds(vb + lane * 8, dst + kTile);
        copy16_global_to_lds(vb + 512 + lane * 8, dst + kTile + 512);
    };
    issue_group(0);
    const PairOrder po = pair_order(ip, T, N1, lane, order[wave]);
    const int mine = po.mine;
    const int steps_both = po.n_both / 2, steps_only = (T - po.n_both) / 2, n_steps = steps_both + 2 * steps_only;

    DqSide sd[2];
    dq_begin(sd[0], a, delta, dor, bh, b, h, g, lane);
    dq_begin(sd[1], a, delta, dor, bh, b, h, g + 1, lane);

    // (two groups per trip: the buffer a group sits in is then a constant and every LDS address a lane-invariant
    // base plus an immediate)
    auto shared_group = [&](int grp, const bf16* blk) __attribute__((always_inline)) {
        wait_vm0();
        __syncthreads();
        const float w = __builtin_amdgcn_logf(a.lvl[shared_level(a.lvl, a.levels, kGroup * grp)].w);   // log2
        PairR r0;
        PairT t0;
        read_k_r(r0, blk, blk + 2 * kTile, lane);
        read_v_r(r0, blk + kTile, blk + 3 * kTile, lane);
        read_k_t(t0, blk, blk + 2 * kTile, lane);
        dq_pair_of_blocks(sd[0], r0, t0, w);
        dq_pair_of_blocks(sd[1], r0, t0, w);
        read_k_r(r0, blk + 4 * kTile, blk + 6 * kTile, lane);
        read_v_r(r0, blk + 5 * kTile, blk + 7 * kTile, lane);
        read_k_t(t0, blk + 4 * kTile, blk + 6 * kTile, lane);
        if (grp + 1 < n_groups) issue_group(grp + 1);
        dq_pair_of_blocks(sd[0], r0, t0, w);
        dq_pair_of_blocks(sd[1], r0, t0, w);
    };
    for (int grp = 0; grp < n_groups; grp += 2) {
        shared_group(grp, sh0);
        if (grp + 1 < n_groups) shared_group(grp + 1, sh0 + kGroup * (2 * kTile));
    }
    __syncthreads();

    bf16* const priv = sh0 + wave * (4 * kTile);
    PairR ra, rb;
    auto fetch = [=](int t, PairR& dst) __attribute__((always_inline)) {
        bf16* slot = priv + (t & 1) * (2 * kTile);
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int blk = __builtin_amdgcn_readlane(mine, 2 * t + j);
            const bf16* kb = kr + (int64_t)blk * kTile;
            const bf16* vb = vr + (int64_t)blk * kTile;
            copy16_global_to_lds(kb + lane * 8, slot + j * kTile);
            copy16_global_to_lds(kb + 512 + lane * 8, slot + j * kTile + 512);
            dst.v[j][0] = ld16(vb + lane * 8);
            dst.v[j][1] = ld16(vb + 512 + lane * 8);
        }
    };
    auto work = [&](int t, PairR& cur, PairR& nxt) __attribute__((always_inline)) {
        wait_vm0();
        const bf16* slot = priv + (t & 1) * (2 * kTile);
        PairT tt;
        read_k_r(cur, slot, slot + kTile, lane);
        read_k_t(tt, slot, slot + kTile, lane);
        if (t + 1 < n_steps) fetch(t + 1, nxt);
        if (t < steps_both + steps_only) dq_pair_of_blocks(sd[0], cur, tt, 0.f);
        if (t < steps_both || t >= steps_both + steps_only) dq_pair_of_blocks(sd[1], cur, tt, 0.f);
    };
    fetch(0, ra);
    for (int t = 0; t < n_steps; t += 2) {
        work(t, ra, rb);
        if (t + 1 < n_steps) work(t + 1, rb, ra);
    }
    dq_end(sd[0], a, b, h, g, lane);
    dq_end(sd[1], a, b, h, g + 1, lane);
}

// ---------------------------------------------------------------------------------------
// K-side gradients.  A "unit" is 16 key rows (a fine K block, 16 pooled tokens of one coarse
// block, or 16 tokens of the dense coarsest level).  Three kernels: attn_kside_kernel walks the
// transposed selection of the fine blocks (unit-major: a unit and the list of query blocks that
// selected it), attn_kside_group_kernel the pooled levels under an ancestor's selection
// (query-group-major), attn_kside_dense_kernel the dense coarsest level.
// ---------------------------------------------------------------------------------------

// Optional last step of the fine dK / dV: add the pooled gradients the token's block received
// (what the backward of the two mean pools and autograd's accumulation do in the reference:
// every sum and every division by 16 rounded to bf16) and rotate dK back through the RoPE.
struct PoolFold {
    const bf16* gk[LLSA_MAX_LEVELS];              // gradients of the pooled k per level, (BH, N/16^l, 64); depth == 0: no folding
    const bf16* gv[LLSA_MAX_LEVELS];
    const bf16* freq;                             // (N, 64) or nullptr
    int depth;                                    // pooled levels to fold in
};
// What a token receives from its pooled ancestors, level by level, coarsest first (pool_bwd_accum_kernel applied down the
// chain): below = the running sum of the level above, g = the gradient of this level's own pooled token.
__device__ __forceinline__ bf16x4 fold_step(bf16x4 g, bf16x4 below) {
#pragma clang fp contract(off)
#pragma unroll
    for (int e = 0; e < 4; e++) g[e] = (bf16)((float)g[e] + rn_bf16((float)below[e] * 0.0625f));
    return g;
}
// x: four channels of one token; c: the same channels of the chain's sum at its level-1 ancestor; f: their [sin, cos] entries
__device__ __forceinline__ bf16x4 fold_math(bf16x4 x, bf16x4 c, bool has_f, bf16x4 f) {
    x = fold_step(x, c);
    return has_f ? rope_bwd4(x, f) : x;
}
// x: channels c0..c0+3 of token `tok` of (b,h) `bh`; which = 0 for dK, 1 for dV
__device__ __forceinline__ bf16x4 fold_pooled(bf16x4 x, const PoolFold& f, int which, int64_t bh, int N, int tok, int c0) {
    bf16x4 acc = x;
#pragma nounroll
    for (int l = f.depth - 1; l >= 0; l--) {
        const int sh = 4 * (l + 1);
        const bf16x4 g = ld8((which ? f.gv[l] : f.gk[l]) + (bh * (N >> sh) + (tok >> sh)) * kD + c0);
        acc = (l == f.depth - 1) ? g : fold_step(g, acc);
    }
    const bool rot = which == 0 && f.freq != nullptr;
    bf16x4 fr = x;
    if (rot) fr = ld8(f.freq + (int64_t)tok * kD + c0);
    return fold_math(x, acc, rot, fr);
}
constexpr int kFoldRows = 2 * LLSA_MAX_LEVELS * kD;   // LDS copy of a unit's fold operands: per level its dk and dv row, then 16 freq rows
constexpr int kFoldElems = kFoldRows + kBlk * kD;

struct KSideParams {
    const bf16* qr;  const bf16* dor;             // R tiles of q and dO, (BH, N1, 1024)
    const float* lse; const float* delta;         // (BH, N)
    const bf16* kk;  const bf16* vv;              // R tiles the unit's 16 key rows come from, (BH, n_units, 1024)
    const int* off;  const int* flat;             // CSR of the transposed selection (per K block)
    const int* work;                              // work list over that CSR (see transpose.hip)
    bf16* dk; int64_t sdkb, sdkh, sdkn;           // bf16 outputs
    bf16* dv; int64_t sdvb, sdvh, sdvn;
    f32x4* part;                                  // fp32 partials: slots (fine pass) or chunks (dense pass)
    int H, N, n_units, chunk_len;
    int64_t flat_stride;                          // entries of `flat` per (b,h)
    int64_t work_stride;                          // ints of `work` per (b,h)
    int64_t slot_stride;                          // partial slots per (b,h)
    float w;
    PoolFold fold;                                // fine pass only
};

// Two query blocks against the unit's 16 key rows, operands out of a wave-private piece of LDS: `stage` holds the
// R tiles of Q and dO of the two blocks (block u: Q at 2u, dO at 2u + 1), `stats` their lse and delta rows.  The tiles
// are read twice, plainly as the A operands of S = Q.K^T and dP = dO.V^T and with the transposing read as the T
// operands of dV^T += dO^T.P and dK^T += Q^T.dS.
struct KsideOperands {
    bf16x8 aq[2][2], ag[2][2];
    bf16x4 tq[2][4], tg[2][4];
    f32x4 l4[2], d4[2];
};
__device__ __forceinline__ void kside_read(KsideOperands& o, const bf16* stage, const float* stats, int lane) {
    const int quad = lane >> 4;
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const bf16* q = stage + (2 * u) * kTile;
        const bf16* g = stage + (2 * u + 1) * kTile;
        o.aq[u][0] = lds_ld16(q + lane * 8);
        o.aq[u][1] = lds_ld16(q + 512 + lane * 8);
        o.ag[u][0] = lds_ld16(g + lane * 8);
        o.ag[u][1] = lds_ld16(g + 512 + lane * 8);
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
            o.tq[u][dt] = lds_t_operand(q, dt, lane);
            o.tg[u][dt] = lds_t_operand(g, dt, lane);
        }
        o.l4[u] = *reinterpret_cast<const f32x4*>(stats + u * 32 + quad * 4);
        o.d4[u] = *reinterpret_cast<const f32x4*>(stats + u * 32 + 16 + quad * 4);
    }
}
__device__ __forceinline__ void kside_pair(f32x4 dk[4], f32x4 dv[4], const bf16x8 bk[2], const bf16x8 bv[2], const KsideOperands& o,
                                           bool second_valid) {
    bf16x8 bp, bds;
#pragma unroll
    for (int u = 0; u < 2; u++) {
        f32x4 s = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
        s = mfma_bf16(o.aq[u][0], bk[0], s);
        s = mfma_bf16(o.aq[u][1], bk[1], s);
        dp = mfma_bf16(o.ag[u][0], bv[0], dp);
        dp = mfma_bf16(o.ag[u][1], bv[1], dp);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float pe = exp2_fast(fmaf(s[e], kScaleLog2e, -o.l4[u][e] * kLog2e));
            if (u == 1 && !second_valid) pe = 0.f;
            bp[u * 4 + e] = (bf16)pe;
            bds[u * 4 + e] = (bf16)(pe * (dp[e] - o.d4[u][e]));
        }
    }
#pragma unroll
    for (int dt = 0; dt < 4; dt++) {
        dv[dt] = mfma_bf16(cat(o.tg[0][dt], o.tg[1][dt]), bp, dv[dt]);
        dk[dt] = mfma_bf16(cat(o.tq[0][dt], o.tq[1][dt]), bds, dk[dt]);
    }
}

// A partial sum of one unit (16 key rows x 64 channels, dK and dV) is kept in the MFMA
// accumulator layout: 8 f32x4 registers per lane (4 channel tiles of dK, then 4 of dV).
__device__ __forceinline__ f32x4* part_slot(f32x4* part, int64_t slot) { return part + slot * (8 * kWave); }

// One work item of the fine pass: a key block and a piece (at most fine_chunk(N) <= LLSA_CHUNK_FINE_MAX entries) of its list.
// One wave = one workgroup per item (items differ a lot in length; a wave that shared its workgroup
// with a longer one would keep its registers and LDS allocated while idle).
__global__ __launch_bounds__(64) void attn_kside_kernel(KSideParams p) {
    __shared__ __align__(16) bf16 stage[4 * kTile];           // 2 query blocks x {Q, dO} R tiles
    __shared__ __align__(16) float stats[64];                 // their lse and delta rows
    __shared__ __align__(16) bf16 fold_buf[kFoldElems];
    const int lid = xcd_logical_id();
    const int item = lid % (int)gridDim.x;
    const int bh = lid / (int)gridDim.x;
    const int lane = threadIdx.x & 63;
    const int N1 = p.N / kBlk;
    const int b = bh / p.H, h = bh % p.H;
    const int r = lane & 15, quad = lane >> 4;

    // which 16 key rows, which part of their query-block list, and where the result goes
    int unit, start, cnt;
    int64_t slot = -1;                                        // >= 0: write an fp32 partial
    const int* fl = nullptr;
    {
        // the item's record is fetched together with the count it is checked against (the grid never
        // exceeds the list's storage): the wave knows its key rows and entries after one round trip
        const int* work = p.work + (int64_t)bh * p.work_stride;
        const int n_items = work[0];
        const int* rec = work + 4 + 4 * item;
        unit = rec[0];
        start = rec[1];
        cnt = rec[2];
        const int sl = rec[3];
        if (item >= n_items) return;
        if (sl >= 0) slot = (int64_t)bh * p.slot_stride + sl;
        fl = p.flat + (int64_t)bh * p.flat_stride;
    }
    // What the fold on the way out needs (the unit's pooled-gradient rows, its tokens' RoPE entries)
    // is copied into LDS now, without registers, so that no load waits at the end of the wave.
    const bool folding = p.fold.depth > 0 && slot < 0;
    if (folding) {
        const int row = lane >> 3, piece = lane & 7;          // rows: dk, dv of level 1, of level 2, ...; 8 x 16 bytes each
        if (row < 2 * p.fold.depth) {
            const int lvl = row >> 1;
            int n = N1, u = unit;
            for (int l = 0; l < lvl; l++) {
                n /= kBlk;
                u /= kBlk;
            }
            const bf16* src = ((row & 1) ? p.fold.gv[lvl] : p.fold.gk[lvl]) + ((int64_t)bh * n + u) * kD;
            copy16_global_to_lds(src + piece * 8, fold_buf);
        }
        if (p.fold.freq != nullptr) {
            const bf16* fr = p.fold.freq + (int64_t)unit * kBlk * kD;
            copy16_global_to_lds(fr + lane * 8, fold_buf + kFoldRows);
            copy16_global_to_lds(fr + 512 + lane * 8, fold_buf + kFoldRows + 512);
        }
    }
    // The item's list entries (at most LLSA_CHUNK_FINE_MAX query blocks) are fetched once, entry i into lane i % 64 of
    // register i / 64, and handed out with readlane: the walk below then has no load that depends on a load.
    constexpr int kEntryRegs = LLSA_CHUNK_FINE_MAX / kWave;
    int mine[kEntryRegs];
#pragma unroll
    for (int k = 0; k < kEntryRegs; k++) mine[k] = (k * kWave + lane < cnt) ? fl[start + k * kWave + lane] : 0;
    auto entry = [&](int i) -> int {                          // i is wave-uniform
        int v = __builtin_amdgcn_readlane(mine[0], i & (kWave - 1));
#pragma unroll
        for (int k = 1; k < kEntryRegs; k++) {
            const int o = __builtin_amdgcn_readlane(mine[k], i & (kWave - 1));
            v = ((i >> 6) == k) ? o : v;
        }
        return clampi(v, 0, N1 - 1);
    };

    f32x4 dk[4], dv[4];
#pragma unroll
    for (int dt = 0; dt < 4; dt++) {
        dk[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        dv[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    {
        bf16x8 bk[2], bv[2];
        const bf16* kp = p.kk + ((int64_t)bh * p.n_units + unit) * kTile + lane * 8;
        const bf16* vp = p.vv + ((int64_t)bh * p.n_units + unit) * kTile + lane * 8;
        bk[0] = ld16(kp);
        bk[1] = ld16(kp + 512);
        bv[0] = ld16(vp);
        bv[1] = ld16(vp + 512);
        const bf16* qrb = p.qr + (int64_t)bh * N1 * kTile;
        const bf16* dorb = p.dor + (int64_t)bh * N1 * kTile;
        const float* lseb = p.lse + (int64_t)bh * p.N;
        const float* dlb = p.delta + (int64_t)bh * p.N;
        // The operands of entries i, i + 1 are copied straight into LDS (no registers) while entries i - 2, i - 1 are
        // worked on: a round reads everything it needs out of LDS first, then starts the next copy into the same
        // place, then does its arithmetic.
        auto fetch = [&](int i) __attribute__((always_inline)) {
            const int g0 = entry(i);
            const int g1 = (i + 1 < cnt) ? entry(i + 1) : g0;
            const bf16* q0 = qrb + (int64_t)g0 * kTile + lane * 8;
            const bf16* d0 = dorb + (int64_t)g0 * kTile + lane * 8;
            const bf16* q1 = qrb + (int64_t)g1 * kTile + lane * 8;
            const bf16* d1 = dorb + (int64_t)g1 * kTile + lane * 8;
            copy16_global_to_lds(q0, stage);
            copy16_global_to_lds(q0 + 512, stage + 512);
            copy16_global_to_lds(d0, stage + kTile);
            copy16_global_to_lds(d0 + 512, stage + kTile + 512);
            copy16_global_to_lds(q1, stage + 2 * kTile);
            copy16_global_to_lds(q1 + 512, stage + 2 * kTile + 512);
            copy16_global_to_lds(d1, stage + 3 * kTile);
            copy16_global_to_lds(d1 + 512, stage + 3 * kTile + 512);
            if (lane < 16) {                                  // four floats a lane: lse g0, delta g0, lse g1, delta g1
                const float* src = ((lane & 4) ? dlb : lseb) + ((lane & 8) ? g1 : g0) * kBlk + (lane & 3) * 4;
                copy16_global_to_lds(reinterpret_cast<const bf16*>(src), reinterpret_cast<bf16*>(stats));
            }
        };
        if (cnt > 0) fetch(0);
        for (int i = 0; i < cnt; i += 2) {
            wait_vm0();
            KsideOperands o;
            kside_read(o, stage, stats, lane);
            wait_all_mem();                                   // every lane has its operands: the next copy may land
            __builtin_amdgcn_wave_barrier();
            if (i + 2 < cnt) fetch(i + 2);
            kside_pair(dk, dv, bk, bv, o, i + 1 < cnt);
        }
    }

    if (slot >= 0) {
        f32x4* ps = part_slot(p.part, slot);
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
            ps[dt * kWave + lane] = dk[dt];
            ps[(4 + dt) * kWave + lane] = dv[dt];
        }
        return;
    }
    bf16* kp = p.dk + b * p.sdkb + h * p.sdkh + (int64_t)(unit * kBlk + r) * p.sdkn + quad * 4;
    bf16* vp = p.dv + b * p.sdvb + h * p.sdvh + (int64_t)(unit * kBlk + r) * p.sdvn + quad * 4;
    if (folding) {
        wait_vm0();                                           // the copies into fold_buf (long since done)
        // the chain of pooled levels collapses into one row for dk and one for dv, left where level 1's rows were:
        // lane (which, four channels) reads its channels of every level and is the only one to write them
        if (lane < 32) {
            const int which = lane >> 4, c0 = (lane & 15) * 4;
            bf16x4 acc = lds_ld8(fold_buf + (2 * (p.fold.depth - 1) + which) * kD + c0);
#pragma nounroll
            for (int l = p.fold.depth - 2; l >= 0; l--) acc = fold_step(lds_ld8(fold_buf + (2 * l + which) * kD + c0), acc);
            lds_st8(fold_buf + which * kD + c0, acc);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
#pragma unroll
    for (int dt = 0; dt < 4; dt++) {
        bf16x4 ok = cvt4(dk[dt] * kScale), ov = cvt4(dv[dt]);
        if (folding) {
            const int c0 = dt * 16 + quad * 4;
            ok = fold_math(ok, lds_ld8(fold_buf + c0), p.fold.freq != nullptr, lds_ld8(fold_buf + kFoldRows + r * kD + c0));
            ov = fold_math(ov, lds_ld8(fold_buf + kD + c0), false, ov);
        }
        st8(kp + dt * 16, ok);
        st8(vp + dt * 16, ov);
    }
}

// ---------------------------------------------------------------------------------------
// Dense coarsest level.  Every unit (16 pooled tokens) meets every query block, so the Q / dO
// tiles are the same for all units: a workgroup takes 4 * UPW units (UPW per wave) and one piece
// of the query range and streams that piece through LDS, a pair of query blocks (8 KB) per
// round, once for all of its units.  The more units a workgroup holds, the fewer times the whole
// of Q and dO is streamed through the chip: with many coarsest tokens (long sequences) that
// stream is what the pass costs.
// The stream is three rounds deep: the tiles of round t + 3 are requested from memory (every wave a
// quarter, into registers) while those of round t + 1 move from registers into the other LDS buffer
// and round t is worked on, so a tile has two rounds of arithmetic to arrive.  (Copies straight
// into LDS cannot be run ahead like that: the compiler waits for all of them before any LDS read.)
// Each wave ends with the partial sums of its units over this piece of the range.
// ---------------------------------------------------------------------------------------
constexpr int kDenseWaves = 4;                    // waves per workgroup

template <int UPW>
__global__ __launch_bounds__(64 * kDenseWaves) void attn_kside_dense_kernel(KSideParams p) {
    __shared__ __align__(16) bf16 sh[2][4 * kTile];           // per pair: Q0, dO0, Q1, dO1 as R tiles
    __shared__ __align__(16) float sh_stats[2][64];           // per pair: lse of its 32 queries, then delta
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int quad = lane >> 4;
    const int N1 = p.N / kBlk;
    // Workgroups that stream the same piece of the query range (one per group of units) get neighbouring logical ids,
    // which xcd_logical_id keeps on one XCD: the piece then comes out of that XCD's L2 for all but the first of them.
    const int unit_groups = p.n_units / (kDenseWaves * UPW);
    const int lid = xcd_logical_id();                          // grid: (unit_groups * chunks, BH)
    const int piece = (lid % (int)gridDim.x) / unit_groups;
    const int bh = lid / (int)gridDim.x;
    const int unit0 = (((lid % (int)gridDim.x) % unit_groups) * kDenseWaves + wave) * UPW;   // + UPW <= n_units (the plan sees to it)
    const int start = piece * p.chunk_len;
    const int n_pairs = min(p.chunk_len, N1 - start) / 2;     // even: chunk_len and N1 are multiples of 4
    if (n_pairs <= 0) return;                                 // uniform over the workgroup
    const bf16* qrb = p.qr + ((int64_t)bh * N1 + start) * kTile;
    const bf16* dorb = p.dor + ((int64_t)bh * N1 + start) * kTile;
    const float* lseb = p.lse + (int64_t)bh * p.N + start * kBlk;
    const float* dlb = p.delta + (int64_t)bh * p.N + start * kBlk;

    // wave w moves tile w of a pair's four (query block w/2; Q for even w, dO for odd w); the first 16 lanes of wave 0
    // also its 64 statistics.  Rounds past the end re-read the last pair (no branch around loads).
    struct Stage { bf16x8 a, b; f32x4 s; };
    const bool stat_lane = wave == 0 && lane < 16;
    auto request = [=](int t, Stage& st) __attribute__((always_inline)) {
        t = min(t, n_pairs - 1);
        const bf16* src = ((wave & 1) ? dorb : qrb) + (int64_t)(2 * t + (wave >> 1)) * kTile;
        st.a = ld16(src + lane * 8);
        st.b = ld16(src + 512 + lane * 8);
        // (every lane of every wave loads, lanes 16.. the same as lane % 16: a load inside a branch makes the compiler lose
        // count of the loads in flight, after which it waits for all of them in every round)
        const int sl = lane & 15;
        st.s = *reinterpret_cast<const f32x4*>((sl < 8 ? lseb : dlb) + 2 * t * kBlk + (sl & 7) * 4);
    };
    auto deposit = [&](int t, const Stage& st) __attribute__((always_inline)) {
        bf16* dst = &sh[t & 1][wave * kTile];
        st16(dst + lane * 8, st.a);
        st16(dst + 512 + lane * 8, st.b);
        if (stat_lane) *reinterpret_cast<f32x4*>(&sh_stats[t & 1][lane * 4]) = st.s;
    };
    Stage s0, s1;
    s0.s = s1.s = f32x4{0.f, 0.f, 0.f, 0.f};
    request(0, s0);
    request(1, s1);
    bf16x8 bk[UPW][2], bv[UPW][2];
#pragma unroll
    for (int j = 0; j < UPW; j++) {
        const bf16* kp = p.kk + ((int64_t)bh * p.n_units + unit0 + j) * kTile + lane * 8;
        const bf16* vp = p.vv + ((int64_t)bh * p.n_units + unit0 + j) * kTile + lane * 8;
        bk[j][0] = ld16(kp);
        bk[j][1] = ld16(kp + 512);
        bv[j][0] = ld16(vp);
        bv[j][1] = ld16(vp + 512);
    }
    deposit(0, s0);
    request(2, s0);
    f32x4 dk[UPW][4], dv[UPW][4];
#pragma unroll
    for (int j = 0; j < UPW; j++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
            dk[j][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
            dv[j][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    // Round t.  The barrier at its top says: buffer t & 1 is filled (every wave deposited its part during round t - 1)
    // and everybody is done reading the other buffer, which this round refills for round t + 1 out of the registers
    // `nxt` -- which then take the request for round t + 3.
    auto round = [&](int t, Stage& nxt) __attribute__((always_inline)) {
        __syncthreads();
        const bf16* b = &sh[t & 1][0];
        bf16x8 aq[2][2], ag[2][2];
        bf16x4 tq[2][4], tg[2][4];
        f32x4 l4[2], d4[2];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            aq[u][0] = lds_ld16(b + (2 * u) * kTile + lane * 8);
            aq[u][1] = lds_ld16(b + (2 * u) * kTile + 512 + lane * 8);
            ag[u][0] = lds_ld16(b + (2 * u + 1) * kTile + lane * 8);
            ag[u][1] = lds_ld16(b + (2 * u + 1) * kTile + 512 + lane * 8);
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                tq[u][dt] = lds_t_operand(b + (2 * u) * kTile, dt, lane);
                tg[u][dt] = lds_t_operand(b + (2 * u + 1) * kTile, dt, lane);
            }
            l4[u] = *reinterpret_cast<const f32x4*>(&sh_stats[t & 1][u * kBlk + quad * 4]);
            d4[u] = *reinterpret_cast<const f32x4*>(&sh_stats[t & 1][32 + u * kBlk + quad * 4]);
        }
        deposit(t + 1, nxt);
        request(t + 3, nxt);
        float nl[2][4];
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) nl[u][e] = -l4[u][e] * kLog2e;
#pragma unroll
        for (int j = 0; j < UPW; j++) {
            bf16x8 bp, bds;
#pragma unroll
            for (int u = 0; u < 2; u++) {
                f32x4 s = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
                s = mfma_bf16(aq[u][0], bk[j][0], s);
                s = mfma_bf16(aq[u][1], bk[j][1], s);
                dp = mfma_bf16(ag[u][0], bv[j][0], dp);
                dp = mfma_bf16(ag[u][1], bv[j][1], dp);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float pe = exp2_fast(fmaf(s[e], kScaleLog2e, nl[u][e]));
                    bp[u * 4 + e] = (bf16)pe;
                    bds[u * 4 + e] = (bf16)(pe * (dp[e] - d4[u][e]));
                }
            }
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                dv[j][dt] = mfma_bf16(cat(tg[0][dt], tg[1][dt]), bp, dv[j][dt]);
                dk[j][dt] = mfma_bf16(cat(tq[0][dt], tq[1][dt]), bds, dk[j][dt]);
            }
        }
    };
    // (two rounds per trip without a branch between them: n_pairs is even, and with a conditional second round the
    // compiler loses count of the loads in flight where the loop closes and waits for all of them)
    for (int t = 0; t < n_pairs; t += 2) {
        round(t, s1);
        round(t + 1, s0);
    }
#pragma unroll
    for (int j = 0; j < UPW; j++) {
        f32x4* ps = part_slot(p.part, ((int64_t)piece * gridDim.y + bh) * p.n_units + unit0 + j);
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
            ps[dt * kWave + lane] = dk[j][dt] * p.w;         // (the weight, left out of the exponentials)
            ps[(4 + dt) * kWave + lane] = dv[j][dt] * p.w;
        }
    }
}

// ---------------------------------------------------------------------------------------
// Pooled levels whose keys come from an ancestor's selection (the level-1 pooled tokens of
// llsa_l2 / llsa_l3 under the parent's coarse blocks, the level-2 pooled tokens of llsa_l3 under
// the grand-parent's), "group-major": a workgroup owns one group of 16 consecutive query blocks
// -- the children of one parent, which all read the same pooled key blocks -- copies their Q and
// dO tiles into LDS once (64 KB) and meets every key block of the group's lists there; a wave
// takes its share of the key blocks, two at a time, and ends each with that block's dK / dV summed
// over the group's 256 queries.  A key block selected by several ancestors receives one such
// partial sum per selecting group, written where kside_reduce_kernel finds the partial sums of a
// key block side by side: at the position the transposed selection gives the (ancestor, entry)
// pair.  Walking the transposed lists instead (key block major, the reference's order,
// sparse_attention_res_2.py:492-575) fetches the 64 KB of a group once per key block that
// selected it, T2 times in all.
// With few tokens on the dense coarsest level its blocks are appended to the lists (every group
// meets all of them), which saves that level a pass of its own over Q and dO.
// ---------------------------------------------------------------------------------------
constexpr int kGroupWaves = 4;
constexpr int kGroupSegs = LLSA_MAX_LEVELS;
constexpr int kGroupMaxBlocks = 64;               // key blocks per group over all its lists (their ids live in one lane each)
constexpr int kGroupDenseMax = 8;                 // dense blocks are appended up to this many
static_assert(LLSA_POOLED_TOPK_MAX + kGroupDenseMax <= kGroupMaxBlocks, "a group's lists must fit one lane per key block");

struct GroupSeg {
    const bf16* kk; const bf16* vv;               // R tiles of this level's pooled k, v: (BH, n_units, 1024)
    const int* sel;                               // (BH, n_groups >> owner_shift, cnt) blocks selected by the group's ancestor;
                                                  // nullptr: blocks 0..cnt-1 (dense level)
    const int* inv;                               // (BH, n_groups >> owner_shift, cnt) position of each entry in the transposed selection
    bf16x8* part;                                 // partial sums, the accumulators of part_slot rounded to bf16, two registers (16 bytes)
                                                  // per lane side by side: slot = [4 register pairs][64 lanes] bf16x8.  The
                                                  // group-major pass writes one per (group, key block), 8 KB each in fp32, which at
                                                  // 16384 tokens is more memory traffic than everything else the pass moves; a group's
                                                  // sum over its 256 queries is taken in fp32 and rounded once (2^-9 relative), and the
                                                  // reduction adds the rounded sums of a key block's groups in fp32
    int n_units, owner_shift, cnt;
    int64_t slots;                                // partial slots per (b,h) (sparse) -- positions are clamped into them
    float w;
};
struct GroupParams {
    const bf16* qr; const bf16* dor;              // R tiles of q and dO, (BH, N1, 1024)
    const float* lse; const float* delta;         // (BH, N)
    int H, N, n_segs, n_blocks;
    GroupSeg seg[kGroupSegs];
};

struct GroupStats { f32x4 l[2], d[2]; };

// UPW key blocks against the group's 16 query blocks, two query blocks per step, operands out of LDS.
template <int UPW>
__device__ __forceinline__ void group_pass(const bf16x8 (&bk)[2][2], const bf16x8 (&bv)[2][2], const float (&w)[2], bf16x8* const (&dst)[2],
                                           const bf16* shq, const bf16* shg, const float* lseb, const float* dlb, int lane) {
    const int quad = lane >> 4;
    f32x4 dk[UPW][4], dv[UPW][4];
#pragma unroll
    for (int j = 0; j < UPW; j++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
            dk[j][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
            dv[j][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    auto load_stats = [=](int t, GroupStats& st) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            st.l[u] = *reinterpret_cast<const f32x4*>(lseb + (2 * t + u) * kBlk + quad * 4);
            st.d[u] = *reinterpret_cast<const f32x4*>(dlb + (2 * t + u) * kBlk + quad * 4);
        }
    };
    auto step = [&](int t, const GroupStats& cur) __attribute__((always_inline)) {
        bf16x8 aq[2][2], ag[2][2];
        bf16x4 tq[2][4], tg[2][4];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const bf16* q = shq + (2 * t + u) * kTile;
            const bf16* g = shg + (2 * t + u) * kTile;
            aq[u][0] = lds_ld16(q + lane * 8);
            aq[u][1] = lds_ld16(q + 512 + lane * 8);
            ag[u][0] = lds_ld16(g + lane * 8);
            ag[u][1] = lds_ld16(g + 512 + lane * 8);
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                tq[u][dt] = lds_t_operand(q, dt, lane);
                tg[u][dt] = lds_t_operand(g, dt, lane);
            }
        }
        float nl[2][4];
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
            for (int e = 0; e < 4; e++) nl[u][e] = -cur.l[u][e] * kLog2e;
#pragma unroll
        for (int j = 0; j < UPW; j++) {
            bf16x8 bp, bds;
#pragma unroll
            for (int u = 0; u < 2; u++) {
                f32x4 sc = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
                sc = mfma_bf16(aq[u][0], bk[j][0], sc);
                sc = mfma_bf16(aq[u][1], bk[j][1], sc);
                dp = mfma_bf16(ag[u][0], bv[j][0], dp);
                dp = mfma_bf16(ag[u][1], bv[j][1], dp);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float pe = exp2_fast(fmaf(sc[e], kScaleLog2e, nl[u][e]));   // (the weight multiplies the sums below)
                    bp[u * 4 + e] = (bf16)pe;
                    bds[u * 4 + e] = (bf16)(pe * (dp[e] - cur.d[u][e]));
                }
            }
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                dv[j][dt] = mfma_bf16(cat(tg[0][dt], tg[1][dt]), bp, dv[j][dt]);
                dk[j][dt] = mfma_bf16(cat(tq[0][dt], tq[1][dt]), bds, dk[j][dt]);
            }
        }
    };
    GroupStats sa, sb;
    load_stats(0, sa);
#pragma unroll 1
    for (int t = 0; t < kBlk / 2; t += 2) {
        load_stats(t + 1, sb);
        step(t, sa);
        load_stats((t + 2) & (kBlk / 2 - 1), sa);             // (the last one re-reads step 0: no branch around loads)
        step(t + 1, sb);
    }
    // The partial sums of this pass leave as bf16 (see GroupSeg::part): the sum over the group's 256 queries was
    // taken in fp32, and the result the reduction makes of them is a bf16 tensor.
#pragma unroll
    for (int j = 0; j < UPW; j++)
#pragma unroll
        for (int pr = 0; pr < 2; pr++) {                      // registers 2 pr, 2 pr + 1 of dK, then of dV: 16 bytes a lane and store
            dst[j][pr * kWave + lane] = cat(cvt4(dk[j][2 * pr] * w[j]), cvt4(dk[j][2 * pr + 1] * w[j]));
            dst[j][(2 + pr) * kWave + lane] = cat(cvt4(dv[j][2 * pr] * w[j]), cvt4(dv[j][2 * pr + 1] * w[j]));
        }
}

__global__ __launch_bounds__(64 * kGroupWaves, 2) void attn_kside_group_kernel(GroupParams p) {
    __shared__ __align__(16) bf16 sh[2][kBlk * kTile];        // R tiles of the group's 16 query blocks: Q, then dO
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int N1 = p.N / kBlk;
    const int lid = xcd_logical_id();
    const int G = lid % (int)gridDim.x;                        // group of query blocks 16 G .. 16 G + 15
    const int bh = lid / (int)gridDim.x;
    const int n_groups = (int)gridDim.x;

    {   // 32 KB of Q tiles and 32 KB of dO tiles, contiguous in memory, 1 KB per wave and copy
        const bf16* qsrc = p.qr + ((int64_t)bh * N1 + (int64_t)G * kBlk) * kTile;
        const bf16* gsrc = p.dor + ((int64_t)bh * N1 + (int64_t)G * kBlk) * kTile;
#pragma unroll
        for (int i = 0; i < 2 * kBlk / kGroupWaves; i++) {
            const int piece = i * kGroupWaves + wave;
            copy16_global_to_lds(qsrc + piece * 512 + lane * 8, &sh[0][piece * 512]);
            copy16_global_to_lds(gsrc + piece * 512 + lane * 8, &sh[1][piece * 512]);
        }
    }
    // Key block j of the group's lists lives in lane j: which tile, which weight, where its partial sum goes.
    int my_unit = 0, my_seg = 0;
    int64_t my_slot = 0;
    {
        int j = lane, sgi = 0;
        while (sgi < p.n_segs - 1 && j >= p.seg[sgi].cnt) {
            j -= p.seg[sgi].cnt;
            sgi++;
        }
        const GroupSeg& sg = p.seg[sgi];
        if (lane < p.n_blocks) {
            my_seg = sgi;
            if (sg.sel != nullptr) {
                const int64_t e = ((int64_t)bh * (n_groups >> sg.owner_shift) + (G >> sg.owner_shift)) * sg.cnt + j;
                my_unit = clampi(sg.sel[e], 0, sg.n_units - 1);
                const int64_t pos = ((int64_t)clampi(sg.inv[e], 0, (int)((sg.slots >> sg.owner_shift) - 1)) << sg.owner_shift) +
                                    (G & ((1 << sg.owner_shift) - 1));
                my_slot = (int64_t)bh * sg.slots + pos;
            } else {
                my_unit = j;
                my_slot = ((int64_t)G * gridDim.y + bh) * sg.n_units + j;      // [group][bh][unit]: what the dense reduction walks
            }
        }
    }
    const float* lseb = p.lse + (int64_t)bh * p.N + (int64_t)G * kBlk * kBlk;
    const float* dlb = p.delta + (int64_t)bh * p.N + (int64_t)G * kBlk * kBlk;
    // this wave's key blocks: a contiguous share, taken two at a time (the last alone if the share is odd)
    const int per = (p.n_blocks + kGroupWaves - 1) / kGroupWaves;
    const int lo = min(wave * per, p.n_blocks), hi = min(lo + per, p.n_blocks);

    bf16x8 bk[2][2], bv[2][2];
    float w[2];
    bf16x8* dst[2];
    auto fetch = [&](int j, int u) __attribute__((always_inline)) {    // K, V tiles of key block j into register set u
        const int sgi = __builtin_amdgcn_readlane(my_seg, j);
        const int unit = __builtin_amdgcn_readlane(my_unit, j);
        const int slo = __builtin_amdgcn_readlane((int)(my_slot & 0xffffffff), j), shi = __builtin_amdgcn_readlane((int)(my_slot >> 32), j);
        const GroupSeg& sg = p.seg[sgi];
        const bf16* kp = sg.kk + ((int64_t)bh * sg.n_units + unit) * kTile + lane * 8;
        const bf16* vp = sg.vv + ((int64_t)bh * sg.n_units + unit) * kTile + lane * 8;
        bk[u][0] = ld16(kp);
        bk[u][1] = ld16(kp + 512);
        bv[u][0] = ld16(vp);
        bv[u][1] = ld16(vp + 512);
        w[u] = sg.w;
        dst[u] = sg.part + (((int64_t)(unsigned)slo) | ((int64_t)shi << 32)) * (4 * kWave);
    };
    if (lo < hi) fetch(lo, 0);
    if (lo + 1 < hi) fetch(lo + 1, 1);
    wait_vm0();
    __syncthreads();                                          // the copies into LDS are everybody's
    for (int j = lo; j < hi; j += 2) {
        const bool two = j + 1 < hi;
        if (j != lo) {
            fetch(j, 0);
            if (two) fetch(j + 1, 1);
        }
        if (two) group_pass<2>(bk, bv, w, dst, &sh[0][0], &sh[1][0], lseb, dlb, lane);
        else group_pass<1>(bk, bv, w, dst, &sh[0][0], &sh[1][0], lseb, dlb, lane);
    }
}

// Finishes the units whose list was cut into several pieces: the result is the sum of the
// unit's partial slots, added in chunk order, so it does not depend on scheduling.  One launch
// serves the three K-side passes.
struct ReduceJob {
    const f32x4* part;       // fp32 partial sums, or, with half_part, the bf16 ones of the group-major pass (as bf16x4)
    int half_part;
    const int* off;          // CSR offsets (list-driven jobs) or nullptr (dense job)
    const int* work;         // work list (fine job); nullptr with `off`: the partial sums of unit u are slots
                             // [off[u] << csr_shift, off[u + 1] << csr_shift) (group-major pooled jobs)
    int csr_shift;
    bf16* dk; int64_t sdkb, sdkh, sdkn;
    bf16* dv; int64_t sdvb, sdvh, sdvn;
    int n_units, chunk, max_units;       // max_units: upper bound of units this job can have per (b,h)
    int64_t work_stride, slot_stride;
    int n_chunks;            // dense job: partials per unit, at stride BH * n_units slots
    PoolFold fold;           // fine job only
};
struct ReduceParams {
    ReduceJob job[LLSA_MAX_LEVELS + 1];
    int n_jobs, H, N;
};

// Unit positions per job and (b,h) that are walked in parallel: a quarter of the most units the job can have,
// between 32 and 256.  Usually a few per cent of the units have several pieces, and every position beyond
// them is a pair of workgroups that starts, reads one record and leaves (at 256 positions for a job of at
// most 257 units that cost 4 us per launch).
__host__ __device__ inline int reduce_slots(int max_units) {
    if (max_units <= 32) return max_units;
    const int q = max_units / 4;
    return q < 32 ? 32 : (q > 256 ? 256 : q);
}

__global__ __launch_bounds__(256) void kside_reduce_kernel(ReduceParams rp) {
    // fp32 partial sums: two workgroups per unit; every thread owns one f32x4 of the unit's 8 x 64 accumulator
    // registers and streams that position of all partials, sixteen loads in flight.  bf16 partial sums (the group-major
    // pass): one workgroup per unit, every thread owns a pair of registers (16 bytes a partial, like the fp32 loads), and
    // the two workgroups of a position take alternate units.  Every job has its own range of workgroup pairs
    // (reduce_slots of them), which walk the job's units with that stride: the number of units with several pieces is
    // known only on the device and usually small, and a grid sized for the worst case would be mostly workgroups that
    // start, look and leave.
    const int bh = blockIdx.y, b = bh / rp.H, h = bh % rp.H;
    int u0 = blockIdx.x >> 1, j = 0;
    while (j < rp.n_jobs && u0 >= reduce_slots(rp.job[j].max_units)) {
        u0 -= reduce_slots(rp.job[j].max_units);
        j++;
    }
    if (j >= rp.n_jobs) return;
    const ReduceJob& jb = rp.job[j];
    const int half = jb.half_part;
    const int pos = half ? (int)threadIdx.x : (int)((blockIdx.x & 1) * 256 + threadIdx.x);
    const int reg = half ? 2 * (pos >> 6) : (pos >> 6), lane = pos & 63;     // (half: registers reg, reg + 1)
    const int r = lane & 15, quad = lane >> 4;
    const int dt = reg & 3;
    const int which = reg >> 2;                               // 0: dK, 1: dV
    const int step = reduce_slots(jb.max_units) * (half ? 2 : 1);
    if (half) u0 = 2 * u0 + (int)(blockIdx.x & 1);
    const int* work = jb.work ? jb.work + (int64_t)bh * jb.work_stride : nullptr;
    const int max_items = (int)(jb.work_stride - work_tail_len(jb.n_units) - 4 - 4 * jb.max_units) / 4;
    // the unit's record is fetched together with the count it is checked against (u0 is always
    // inside the list's storage): one memory round trip instead of two
    const int* multi = work ? work + 4 + 4 * max_items : nullptr;
    int rec_unit = 0, rec_first = 0, rec_n = 0;
    if (work != nullptr) {
        rec_unit = multi[4 * u0];
        rec_first = multi[4 * u0 + 1];
        rec_n = multi[4 * u0 + 2];
    }
    const int count = work ? min(work[2], jb.max_units) : jb.n_units;
    for (int u = u0; u < count; u += step) {
        int unit, n;
        int64_t first, stride;
        if (work != nullptr) {
            if (u != u0) {
                rec_unit = multi[4 * u];
                rec_first = multi[4 * u + 1];
                rec_n = multi[4 * u + 2];
            }
            unit = rec_unit;
            n = rec_n;
            first = (int64_t)bh * jb.slot_stride + rec_first;
            stride = 1;
        } else if (jb.off != nullptr) {
            const int* o = jb.off + (int64_t)bh * (jb.n_units + 1) + u;
            const int o0 = o[0], o1 = o[1];
            unit = u;
            n = (o1 - o0) << jb.csr_shift;
            first = (int64_t)bh * jb.slot_stride + ((int64_t)o0 << jb.csr_shift);
            stride = 1;
        } else {
            unit = u;
            n = jb.n_chunks;
            first = (int64_t)bh * jb.n_units + unit;
            stride = (int64_t)gridDim.y * jb.n_units;
        }
        f32x4 acc = {0.f, 0.f, 0.f, 0.f}, acc2 = {0.f, 0.f, 0.f, 0.f};
        if (half) {
            const bf16x8* ps = reinterpret_cast<const bf16x8*>(jb.part) + first * (4 * kWave) + (reg >> 1) * kWave + lane;
            for (int c0 = 0; c0 < n; c0 += 16) {
                bf16x8 v[16];
#pragma unroll
                for (int k = 0; k < 16; k++) v[k] = ps[(int64_t)min(c0 + k, n - 1) * stride * (4 * kWave)];
#pragma unroll
                for (int k = 0; k < 16; k++)
                    if (c0 + k < n) {
                        acc += f32x4{(float)v[k][0], (float)v[k][1], (float)v[k][2], (float)v[k][3]};
                        acc2 += f32x4{(float)v[k][4], (float)v[k][5], (float)v[k][6], (float)v[k][7]};
                    }
            }
        } else {
            const f32x4* ps = jb.part + first * (8 * kWave) + reg * kWave + lane;
            for (int c0 = 0; c0 < n; c0 += 16) {
                f32x4 v[16];
#pragma unroll
                for (int k = 0; k < 16; k++) v[k] = ps[(int64_t)min(c0 + k, n - 1) * stride * (8 * kWave)];
#pragma unroll
                for (int k = 0; k < 16; k++)
                    if (c0 + k < n) acc += v[k];               // chunk order: the sum does not depend on scheduling
            }
        }
        bf16* dst = which ? jb.dv + b * jb.sdvb + h * jb.sdvh + (int64_t)(unit * kBlk + r) * jb.sdvn
                          : jb.dk + b * jb.sdkb + h * jb.sdkh + (int64_t)(unit * kBlk + r) * jb.sdkn;
        bf16x4 out = cvt4(which ? acc : acc * kScale);
        if (jb.fold.depth > 0)
            out = fold_pooled(out, jb.fold, which, bh, rp.N, unit * kBlk + r, dt * 16 + quad * 4);
        st8(dst + quad * 4 + dt * 16, out);
        if (half) st8(dst + quad * 4 + (dt + 1) * 16, cvt4(which ? acc2 : acc2 * kScale));      // (no fold on these jobs)
    }
}

struct DensePlan {
    int n_tok;       // tokens of the dense coarsest level per (b,h)
    int upw;         // units per wave (1 or 2): a workgroup holds 4 * upw units
    int chunks;      // query range split
    int chunk_len;   // query blocks per chunk (a multiple of 4)
    bool merged;     // the dense blocks ride on the group-major pass (one partial sum per group of 16 query blocks)
};

static DensePlan dense_plan(int B, int H, int N, int levels) {
    const int N1 = N / 16;
    DensePlan d;
    d.n_tok = N1;                                             // tokens of pooled level `levels`
    for (int l = 1; l < levels; l++) d.n_tok /= 16;
    const int n_units = d.n_tok / 16;
    // Q and dO are streamed n_units / (4 * upw) times (mostly out of an L2: see the kernel); four units per wave would
    // halve that again but leave one wave per SIMD, which measured slower (1.07 ms against 0.93 ms at N = 262144)
    d.upw = (n_units % 8 == 0 && n_units >= 16) ? 2 : 1;
    const int groups = max(1, n_units / (kDenseWaves * d.upw)) * B * H;   // workgroups per piece of the query range
    // The query range is cut so that the workgroups fill the chip's resident slots (256 CUs x the workgroups the
    // registers allow per CU) a whole number of times, three if there is that much work: a count just above a
    // multiple of the slots leaves a last round in which a few workgroups run alone.
    const int slots = 256 * (d.upw == 2 ? 2 : 3);
    int chunks = 3 * slots / groups;
    if (chunks > N1 / 16) chunks = N1 / 16;
    if (chunks < 1) chunks = 1;
    int len = (N1 + chunks - 1) / chunks;
    len = (len + 3) & ~3;
    d.chunk_len = len;
    d.chunks = (N1 + len - 1) / len;
    d.merged = levels >= 2 && n_units <= kGroupDenseMax;
    if (d.merged) {
        d.chunks = N1 / 16;
        d.chunk_len = 16;
    }
    return d;
}

static int64_t align256(int64_t x) { return (x + 255) & ~(int64_t)255; }
constexpr int64_t kSlotBytes = 8 * kWave * sizeof(f32x4);     // one partial: 16 rows x 64 ch x (dK, dV) fp32

struct BwdWorkspace {
    int64_t delta, dor, part_fine, part_dense, total;
    int64_t part_level[LLSA_MAX_LEVELS];                        // partial sums of pooled level l (below the coarsest) at [l - 1]
    int64_t slots_fine, slots_level[LLSA_MAX_LEVELS];           // per (b,h)
};

// topk[0] = T of the fine blocks, topk[l] = T of pooled level l (l < levels)
static BwdWorkspace bwd_workspace(int B, int H, int N, const int32_t* topk, int levels) {
    const int64_t BH = (int64_t)B * H, N1 = N / 16, N2 = N1 / 16;
    const DensePlan d = dense_plan(B, H, N, levels);
    BwdWorkspace w;
    // a key block has several chunks only if it has more than `chunk` entries, so at most
    // E/chunk such blocks with at most E/chunk + E/chunk chunks in total
    w.slots_fine = 2 * (N1 * topk[0] / fine_chunk(N)) + 2;
    int64_t o = 0;
    w.delta = o;        o += align256(BH * N * 4);
    w.dor = o;          o += align256(BH * N * 64 * 2);
    w.part_fine = o;    o += align256(BH * w.slots_fine * kSlotBytes);
    // group-major pooled passes: one partial sum per (group of 16 query blocks, entry of its ancestor's list)
    for (int l = 1; l <= LLSA_MAX_LEVELS; l++) {
        w.slots_level[l - 1] = (l < levels) ? N2 * topk[l] : 0;
        w.part_level[l - 1] = o;
        o += align256(BH * w.slots_level[l - 1] * kSlotBytes);
    }
    w.part_dense = o;   o += align256((int64_t)d.chunks * BH * (d.n_tok / 16) * kSlotBytes);
    w.total = o;
    return w;
}

}  // namespace llsa

using namespace llsa;

extern "C" int64_t llsa_attn_bwd_workspace_bytes(int B, int H, int N, const int32_t* topk, int levels) {
    if (B <= 0 || H <= 0 || N <= 0 || topk == nullptr || levels < 1 || levels > LLSA_MAX_LEVELS) return -1;
    if (N % coarsest_multiple(levels) != 0) return -1;       // what llsa_attn_bwd asks of N: whole 64-token tiles of the coarsest level
    for (int l = 0; l < levels; l++)
        if (topk[l] <= 0) return -1;
    return bwd_workspace(B, H, N, topk, levels).total;
}

extern "C" int llsa_attn_bwd(const llsa_attn_bwd_args* a, void* stream) {
    LLSA_REQUIRE(a != nullptr, "attn_bwd: null args");
    LLSA_REQUIRE(a->levels >= 1 && a->levels <= LLSA_MAX_LEVELS, "attn_bwd: levels must be 1..%d", LLSA_MAX_LEVELS);
    LLSA_REQUIRE(a->B > 0 && a->H > 0 && a->N > 0, "attn_bwd: bad B/H/N");
    LLSA_REQUIRE(a->dout && a->o && a->lse && a->qr && a->kr && a->vr && a->idx && a->off && a->flat && a->dq && a->dk && a->dv &&
                     a->workspace,
                 "attn_bwd: null tensor");
    LLSA_REQUIRE(a->T >= 4 && a->T % 4 == 0 && a->T <= a->N / 16, "attn_bwd: topk=%d must be a multiple of 4 and <= N/16", a->T);
    const int64_t mult = coarsest_multiple(a->levels);
    LLSA_REQUIRE(a->N % mult == 0, "attn_bwd: %d level(s) need N %% %lld == 0 (N=%d)", a->levels, (long long)mult, a->N);
    int32_t topk[LLSA_MAX_LEVELS] = {a->T, 0, 0, 0};
    int listed = 0;
    int64_t span = 256;
    for (int l = 1; l <= a->levels; l++, span *= 16) {
        const llsa_bwd_level& lv = a->lvl[l - 1];
        LLSA_REQUIRE(lv.kr && lv.vr && lv.dk && lv.dv, "attn_bwd: tensors of level %d missing", l);
        LLSA_REQUIRE(aligned16(lv.kr) && aligned16(lv.vr) && aligned16(lv.dk) && aligned16(lv.dv), "attn_bwd: tensors must be 16-byte aligned");
        LLSA_REQUIRE(lv.w > 0.f && lv.gw > 0.f, "attn_bwd: the weights of level %d must be > 0", l);
        if (l < a->levels) {
            LLSA_REQUIRE(lv.sel && lv.off && lv.inv, "attn_bwd: selection of level %d or its transpose missing", l);
            LLSA_REQUIRE(lv.T >= 4 && lv.T % 4 == 0 && lv.T <= a->N / span, "attn_bwd: topk of level %d (%d) must be a multiple of 4 and <= N/%lld",
                         l, lv.T, (long long)span);
            topk[l] = lv.T;
            listed += lv.T;
        }
    }
    LLSA_REQUIRE(listed <= LLSA_POOLED_TOPK_MAX, "attn_bwd: the topk of the pooled levels together (%d) must not exceed %d", listed,
                 LLSA_POOLED_TOPK_MAX);
    const void* al[] = {a->dout, a->o, a->qr, a->kr, a->vr, a->dq, a->dk, a->dv, a->workspace, a->freq_dq, a->lse};
    for (const void* p : al) LLSA_REQUIRE(aligned16(p), "attn_bwd: tensors must be 16-byte aligned");
    const int64_t st[] = {a->sdob, a->sdoh, a->sdon, a->sob, a->soh, a->son};
    for (int64_t s : st) LLSA_REQUIRE(stride_ok(s), "attn_bwd: input row strides must keep rows 16-byte aligned");
    const int64_t so[] = {a->sdqb, a->sdqh, a->sdqn, a->sdkb, a->sdkh, a->sdkn, a->sdvb, a->sdvh, a->sdvn};
    for (int64_t s : so) LLSA_REQUIRE(s % 4 == 0, "attn_bwd: output row strides must keep rows 8-byte aligned");
    const BwdWorkspace wsp = bwd_workspace(a->B, a->H, a->N, topk, a->levels);
    LLSA_REQUIRE(a->workspace_bytes >= wsp.total, "attn_bwd: workspace too small (%lld < %lld)", (long long)a->workspace_bytes,
                 (long long)wsp.total);
    LLSA_REQUIRE(a->work != nullptr, "attn_bwd: work list missing");

    hipStream_t s = (hipStream_t)stream;
    const int B = a->B, H = a->H, N = a->N, N1 = N / 16, N2 = N1 / 16, BH = B * H, L = a->levels;
    const DensePlan d = dense_plan(B, H, N, L);
    char* ws = (char*)a->workspace;
    float* delta = (float*)(ws + wsp.delta);
    bf16* dor = (bf16*)(ws + wsp.dor);
    const bool fold = a->fold_pooled != 0;
    LLSA_REQUIRE(fold || a->freq_dk == nullptr, "attn_bwd: freq_dk needs fold_pooled");

    const int stages = a->stages ? a->stages : (0x7fffffff & ~LLSA_BWD_NO_REDUCE);
    if (stages & LLSA_BWD_DQ) {
        if (a->T <= kPairMaxTopk && N1 % 8 == 0)
            hipLaunchKernelGGL(attn_dq_pair_kernel, dim3(N1 / 8, BH), dim3(256), 0, s, *a, delta, dor);
        else
            hipLaunchKernelGGL(attn_dq_kernel, dim3((N1 + 3) / 4, BH), dim3(256), 0, s, *a, delta, dor);
    }

    ReduceParams rp;
    rp.n_jobs = 0;
    rp.H = H;
    rp.N = N;
    PoolFold no_fold;
    for (int l = 0; l < LLSA_MAX_LEVELS; l++) no_fold.gk[l] = no_fold.gv[l] = nullptr;
    no_fold.freq = nullptr;
    no_fold.depth = 0;
    auto add_job = [&](const KSideParams& p, int chunk, int max_units, int n_chunks) {
        ReduceJob& j = rp.job[rp.n_jobs++];
        j.part = p.part; j.half_part = 0; j.off = p.off; j.work = p.work; j.csr_shift = 0;
        j.dk = p.dk; j.sdkb = p.sdkb; j.sdkh = p.sdkh; j.sdkn = p.sdkn;
        j.dv = p.dv; j.sdvb = p.sdvb; j.sdvh = p.sdvh; j.sdvn = p.sdvn;
        j.n_units = p.n_units; j.chunk = chunk; j.max_units = max_units;
        j.work_stride = p.work_stride; j.slot_stride = p.slot_stride; j.n_chunks = n_chunks;
        j.fold = p.fold;
    };
    auto run_reduce = [&]() {
        if (stages & LLSA_BWD_NO_REDUCE) rp.n_jobs = 0;       // (profiling: time the K-side kernels alone)
        if (rp.n_jobs == 0) return;
        int slots = 0;
        for (int i = 0; i < rp.n_jobs; i++) slots += reduce_slots(rp.job[i].max_units);
        hipLaunchKernelGGL(kside_reduce_kernel, dim3(slots * 2, BH), dim3(256), 0, s, rp);
        rp.n_jobs = 0;
    };
    KSideParams base;
    base.qr = (const bf16*)a->qr; base.dor = dor;
    base.lse = a->lse; base.delta = delta;
    base.H = H; base.N = N; base.chunk_len = 0;
    base.fold = no_fold;
    // pooled level l: N / 16^l tokens per (b,h), contiguous (B,H,n,64) gradients
    auto level_tokens = [&](int l) {
        int n = N;
        for (int i = 0; i < l; i++) n /= 16;
        return n;
    };

    auto run_fine = [&]() {                                   // dK / dV of the fine tokens
        if (!(stages & LLSA_BWD_DKV)) return;
        KSideParams p = base;
        p.kk = (const bf16*)a->kr; p.vv = (const bf16*)a->vr;
        p.off = a->off; p.flat = a->flat; p.flat_stride = (int64_t)N1 * a->T;
        const int chunk = fine_chunk(N);
        p.work = a->work; p.work_stride = llsa_work_list_len(N1, N1, a->T, chunk);
        p.part = (f32x4*)(ws + wsp.part_fine); p.slot_stride = wsp.slots_fine;
        p.dk = (bf16*)a->dk; p.sdkb = a->sdkb; p.sdkh = a->sdkh; p.sdkn = a->sdkn;
        p.dv = (bf16*)a->dv; p.sdvb = a->sdvb; p.sdvh = a->sdvh; p.sdvn = a->sdvn;
        p.n_units = N1; p.w = 1.f;
        if (fold) {
            for (int l = 0; l < L; l++) {
                p.fold.gk[l] = (const bf16*)a->lvl[l].dk;
                p.fold.gv[l] = (const bf16*)a->lvl[l].dv;
            }
            p.fold.freq = (const bf16*)a->freq_dk;
            p.fold.depth = L;
        }
        const int max_items = N1 * a->T / chunk + N1;
        hipLaunchKernelGGL(attn_kside_kernel, dim3(max_items, BH), dim3(64), 0, s, p);
        add_job(p, chunk, N1 * a->T / chunk + 1, 0);
    };
    // pooled levels under an ancestor's selection, group-major (one launch for all of them, plus the dense level when it is small)
    auto run_groups = [&]() {
        if (L < 2 || !(stages & LLSA_BWD_DPKV1)) return;
        GroupParams g;
        g.qr = (const bf16*)a->qr; g.dor = dor; g.lse = a->lse; g.delta = delta;
        g.H = H; g.N = N; g.n_segs = 0; g.n_blocks = 0;
        auto add_seg = [&](const void* kk, const void* vv, const int* sel, const int* inv, int64_t part_off, int n_units, int shift,
                           int cnt, int64_t slots, float w) {
            GroupSeg& sgm = g.seg[g.n_segs++];
            sgm.kk = (const bf16*)kk; sgm.vv = (const bf16*)vv; sgm.sel = sel; sgm.inv = inv;
            sgm.part = (bf16x8*)(ws + part_off); sgm.n_units = n_units; sgm.owner_shift = shift; sgm.cnt = cnt; sgm.slots = slots; sgm.w = w;
            g.n_blocks += cnt;
        };
        for (int l = 1; l < L; l++) {                         // level l: blocks N / 16^(l+1), one list per 16^(l-1) groups
            const llsa_bwd_level& lv = a->lvl[l - 1];
            add_seg(lv.kr, lv.vr, lv.sel, lv.inv, wsp.part_level[l - 1], level_tokens(l + 1), 4 * (l - 1), lv.T, wsp.slots_level[l - 1], lv.gw);
        }
        if (d.merged && (stages & LLSA_BWD_DENSE))
            add_seg(a->lvl[L - 1].kr, a->lvl[L - 1].vr, nullptr, nullptr, wsp.part_dense, d.n_tok / 16, 0, d.n_tok / 16, 0, a->lvl[L - 1].gw);
        hipLaunchKernelGGL(attn_kside_group_kernel, dim3(N2, BH), dim3(64 * kGroupWaves), 0, s, g);
        for (int l = 1; l < L; l++) {
            const GroupSeg& sgm = g.seg[l - 1];
            const int64_t n = level_tokens(l);
            ReduceJob& j = rp.job[rp.n_jobs++];
            j.part = (const f32x4*)sgm.part; j.half_part = 1; j.off = a->lvl[l - 1].off; j.work = nullptr; j.csr_shift = sgm.owner_shift;
            j.dk = (bf16*)a->lvl[l - 1].dk; j.sdkb = (int64_t)H * n * 64; j.sdkh = n * 64; j.sdkn = 64;
            j.dv = (bf16*)a->lvl[l - 1].dv; j.sdvb = (int64_t)H * n * 64; j.sdvh = n * 64; j.sdvn = 64;
            j.n_units = sgm.n_units; j.chunk = 1; j.max_units = sgm.n_units;
            j.work_stride = 0; j.slot_stride = sgm.slots; j.n_chunks = 0;
            j.fold = no_fold;
        }
    };
    // dense coarsest level: every unit (16 pooled tokens) meets every query block; the query
    // range is cut into d.chunks pieces whose partial sums are added afterwards
    auto run_dense = [&]() {
        if (!(stages & LLSA_BWD_DENSE)) return;
        KSideParams p = base;
        const llsa_bwd_level& lv = a->lvl[L - 1];
        p.kk = (const bf16*)lv.kr; p.vv = (const bf16*)lv.vr;
        p.dk = (bf16*)lv.dk; p.dv = (bf16*)lv.dv;
        p.sdkb = p.sdvb = (int64_t)H * d.n_tok * 64; p.sdkh = p.sdvh = (int64_t)d.n_tok * 64;
        p.w = lv.gw;
        p.sdkn = p.sdvn = 64;
        p.off = nullptr; p.flat = nullptr; p.flat_stride = 0; p.work = nullptr; p.work_stride = 0; p.slot_stride = 0;
        p.part = (f32x4*)(ws + wsp.part_dense);
        p.n_units = d.n_tok / 16; p.chunk_len = d.chunk_len;
        if (d.merged) {                                       // the group-major pass has written one partial sum per group
            add_job(p, 1, p.n_units, d.chunks);
            rp.job[rp.n_jobs - 1].half_part = 1;
            return;
        }
        const dim3 grid(p.n_units / (kDenseWaves * d.upw) * d.chunks, BH), block(64 * kDenseWaves);
        if (d.upw == 2) hipLaunchKernelGGL(HIP_KERNEL_NAME(attn_kside_dense_kernel<2>), grid, block, 0, s, p);
        else hipLaunchKernelGGL(HIP_KERNEL_NAME(attn_kside_dense_kernel<1>), grid, block, 0, s, p);
        add_job(p, 1, p.n_units, d.chunks);
    };

    if (fold) {
        // the fine pass adds the finished pooled gradients on its way out, so they come first
        run_groups();
        run_dense();
        run_reduce();
        run_fine();
        run_reduce();
    } else {
        run_fine();
        run_groups();
        run_dense();
        run_reduce();
    }
    return launch_status("attn_bwd");
}
