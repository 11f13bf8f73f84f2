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
// KV order per query block: (l2) the 16*T2 level-1 pooled tokens inside the parent's selected
// coarse blocks, then every token of the coarsest pooled level, then the T selected 16-token
// blocks of K/V (the reference walks the same set fine blocks first; the order only moves
// roundings).  Pooled segments count with weight w1 / w2: the accumulator and the running sum
// are kept in units of the current segment's weight, converted once at each segment boundary.
#include "llsa_device.h"
#include "llsa_host.h"
#include "../../include/llsa_hip.h"

namespace llsa {

constexpr float kMaxSlack = 8.f;     // log2 units
constexpr int NB = 2;                // 16-key blocks per pipeline step: 32 keys, one K step of the second product

struct SoftmaxState {
    float m2;        // reference point of the exponentials (at most kMaxSlack below the running max), log2 units
    f32x4 acc[4];    // O^T: channel 16*dt + 4*(l/16) + e of query l%16, in units of the current weight
    float lsum;      // this lane's share of the running sum of the query's p
};

// Operands of one step = NB 16-key blocks, as they sit in registers between load and use.
struct KvRegs {
    bf16x8 k[NB][2];     // K rows (R tile): block j, channel half
    bf16x8 v[NB / 2][4]; // V (T tiles of a pair of blocks): channel tile dt, keys 4*(l/16)..+3 of the first block, then of the second
};

// Where one step's blocks live: kb[j] is the R tile of key block j, vtb[j] the T tile of its values.
struct StepDesc {
    const bf16* kb[NB];
    const bf16* vtb[NB];
};

__device__ __forceinline__ void load_step(KvRegs& t, const StepDesc& d, int lane) {
#pragma unroll
    for (int j = 0; j < NB; j++) {
        t.k[j][0] = ld16(d.kb[j] + lane * 8);
        t.k[j][1] = ld16(d.kb[j] + 512 + lane * 8);
    }
    // (the two halves of an operand are loaded one after the other so that they land in adjacent registers)
#pragma unroll
    for (int c = 0; c < NB / 2; c++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
            t.v[c][dt] = cat(ld8(d.vtb[2 * c] + dt * 256 + lane * 4), ld8(d.vtb[2 * c + 1] + dt * 256 + lane * 4));
}

__device__ __forceinline__ void init_state(SoftmaxState& st) {
    st.m2 = 0.f;
    st.lsum = 0.f;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) st.acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// Changes the unit the accumulator and the running sum are kept in (at a boundary between segments of different weight).
__device__ __forceinline__ void rescale(SoftmaxState& st, float f) {
    st.lsum *= f;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) st.acc[dt] *= f;
}

// The exponentials refer to st.m2, which follows the running maximum lazily: it moves only when the maximum
// has grown by more than kMaxSlack (then p <= 2^kMaxSlack, harmless in bf16 and in the fp32 sums), so that the
// accumulator is rescaled a few times per query block instead of at most steps; O = acc / sum and
// lse = m2 + log2(sum) hold for any reference point.  The common path therefore needs no maximum over the quad
// of lanes that share a query: every lane checks its own exponents against the slack, and only when one in the
// wave exceeds it is the reference point moved (for all four lanes of a query alike, by the quad's largest
// exponent).  st.m2 starts at the largest score of the first block (start_reference), so it is always finite.
__device__ __forceinline__ void start_reference(SoftmaxState& st, const bf16x8 bq[2], const KvRegs& t) {
    f32x4 z = {0.f, 0.f, 0.f, 0.f};
    const f32x4 s = mfma_bf16(t.k[0][1], bq[1], mfma_bf16(t.k[0][0], bq[0], z));
    st.m2 = quad_max(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]))) * kScaleLog2e;
}

// x: the exponents of one step (NB blocks) relative to st.m2
__device__ __forceinline__ void exponents(float x[NB][4], const SoftmaxState& st, const bf16x8 bq[2], const KvRegs& t) {
#pragma unroll
    for (int j = 0; j < NB; j++) {
        f32x4 z = {0.f, 0.f, 0.f, 0.f};
        const f32x4 s = mfma_bf16(t.k[j][1], bq[1], mfma_bf16(t.k[j][0], bq[0], z));
#pragma unroll
        for (int e = 0; e < 4; e++) x[j][e] = fmaf(s[e], kScaleLog2e, -st.m2);
    }
}
__device__ __forceinline__ float largest(const float x[NB][4]) {
    float top = x[0][0];
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) top = fmaxf(top, x[j][e]);
    return top;
}
// the rare path: moves the reference point of every query whose largest exponent exceeds the slack
__device__ __forceinline__ void move_reference(SoftmaxState& st, float x[NB][4], float top) {
    top = quad_max(top);
    const float shift = (top > kMaxSlack) ? top : 0.f;
    st.m2 += shift;
    rescale(st, exp2_fast(-shift));
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) x[j][e] -= shift;
}
__device__ __forceinline__ void accumulate(SoftmaxState& st, const float x[NB][4], const KvRegs& t) {
    bf16x8 bp[NB / 2];
    float rs = 0.f;
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float p = exp2_fast(x[j][e]);
            rs += p;
            bp[j >> 1][(j & 1) * 4 + e] = (bf16)p;
        }
    st.lsum += rs;
#pragma unroll
    for (int c = 0; c < NB / 2; c++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
            st.acc[dt] = mfma_bf16(t.v[c][dt], bp[c], st.acc[dt]);
}

__device__ __forceinline__ void compute_step(SoftmaxState& st, const bf16x8 bq[2], const KvRegs& t) {
    float x[NB][4];
    exponents(x, st, bq, t);
    const float top = largest(x);
    if (__ballot(top > kMaxSlack) != 0) move_reference(st, x, top);
    accumulate(st, x, t);
}

// The same step for two query blocks that read the same operands, written as one straight-line piece so that the
// products of one block overlap with the exponentials of the other (one test for the rare path covers both).
__device__ __forceinline__ void compute_step2(SoftmaxState& sa, SoftmaxState& sb, const bf16x8 qa[2], const bf16x8 qb[2], const KvRegs& t) {
    float xa[NB][4], xb[NB][4];
    exponents(xa, sa, qa, t);
    exponents(xb, sb, qb, t);
    const float ta = largest(xa), tb = largest(xb);
    if (__ballot(fmaxf(ta, tb) > kMaxSlack) != 0) {
        move_reference(sa, xa, ta);
        move_reference(sb, xb, tb);
    }
    accumulate(sa, xa, t);
    accumulate(sb, xb, t);
}

// Operands of one step out of the workgroup's LDS copy of shared blocks (4 KB per block: R tile
// of the keys, then T tile of the values).
__device__ __forceinline__ void load_step_lds(KvRegs& t, const bf16* blocks, int lane) {
#pragma unroll
    for (int j = 0; j < NB; j++) {
        t.k[j][0] = lds_ld16(blocks + j * 2 * kTile + lane * 8);
        t.k[j][1] = lds_ld16(blocks + j * 2 * kTile + 512 + lane * 8);
    }
#pragma unroll
    for (int c = 0; c < NB / 2; c++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
            t.v[c][dt] = cat(lds_ld8(blocks + (2 * c) * 2 * kTile + kTile + dt * 256 + lane * 4),
                             lds_ld8(blocks + (2 * c + 1) * 2 * kTile + kTile + dt * 256 + lane * 4));
            __builtin_amdgcn_sched_barrier(0);    // (keeps the two reads one paired LDS read: paired with any other read they need moves)
        }
}

__device__ __forceinline__ void finish_query_block(const llsa_attn_fwd_args& a, const SoftmaxState& st, int bh, int b, int h, int g, int lane) {
    const int r = lane & 15, quad = lane >> 4;
    const float L = quad_sum(st.lsum);
    const float inv = 1.f / L;
    bf16* op = (bf16*)a.o + b * a.sob + h * a.soh + (int64_t)(g * kBlk + r) * a.son + quad * 4;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) st8(op + dt * 16, cvt4(st.acc[dt] * inv));
    if (quad == 0) a.lse[(int64_t)bh * a.N + g * kBlk + r] = (st.m2 + __builtin_amdgcn_logf(L)) * kLn2;
}

// One wave per query block, four consecutive query blocks per workgroup.
//
// The pooled blocks -- the level-1 pooled tokens of the parent's coarse blocks and the coarsest
// level -- are the same for all query blocks of a 256-token parent, hence for the four waves of
// the workgroup: they are fetched once per workgroup, kGroup at a time, straight into LDS (two
// buffers, the next fetch in flight during the arithmetic), and every wave reads its operands
// from there.  The T fine blocks differ from query block to query block: every wave then walks
// its own in steps of NB blocks, the loads of step t+1 issued before the arithmetic of step t
// (two register buffers, ping-pong).  The shared phase comes first because the compiler drains
// the whole vector-memory queue at every wait while a copy into LDS is outstanding, which would
// undo the register ping-pong.  This is what bounds the kernel: without the sharing every wave
// pulls all of its 4 KB per block through the L2, and the L2's bandwidth, not the MFMA, sets the time.
__global__ __launch_bounds__(256, 4) void attn_fwd_kernel(llsa_attn_fwd_args a) {
    static_assert(NB == 2 && kGroup == 4, "the shared phase reads an LDS buffer of four blocks as two steps of two");
    __shared__ __align__(16) bf16 sh[2][kGroup][2 * kTile];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int N1 = a.N / kBlk;
    const int lid = xcd_logical_id();
    const int g = (lid % (int)gridDim.x) * 4 + wave;          // < N1: the host checks N1 % 4 == 0
    const int bh = lid / (int)gridDim.x, b = bh / a.H, h = bh % a.H;

    const bf16* kr = (const bf16*)a.kr + (int64_t)bh * N1 * kTile;
    const bf16* vt = (const bf16*)a.vt + (int64_t)bh * N1 * kTile;
    const int* ip = a.idx + ((int64_t)bh * N1 + g) * a.T;

    // Shared list: for every pooled level below the coarsest the blocks its ancestor group selected (level 1 first),
    // then every block of the coarsest level.  The selected entries of all levels together (at most 64: the host
    // checks) live one per lane, entry i in lane i.
    SharedList sl = shared_list(a.lvl, a.levels, a.N, bh, g, lane);
    bf16* const sh0 = &sh[0][0][0];
    auto issue_group = [&](int grp) __attribute__((always_inline)) {   // this wave brings in block kGroup*grp + wave
        const SharedBlock sb = shared_block(sl, a.lvl, a.levels, a.N, bh, kGroup * grp + wave);
        const bf16* kb = (const bf16*)a.lvl[sb.level].kr + sb.tile;
        const bf16* vb = (const bf16*)a.lvl[sb.level].vt + sb.tile;
        bf16* dst = sh0 + ((grp & 1) * kGroup + wave) * (2 * kTile);
        copy16_global_to_lds(kb + lane * 8, dst);
        copy16_global_to_lds(kb + 512 + lane * 8, dst + 512);
        copy16_global_to_lds(vb + lane * 8, dst + kTile);
        copy16_global_to_lds(vb + 512 + lane * 8, dst + kTile + 512);
    };
    const int n_groups = sl.n_blocks / kGroup;                // every level's count is a multiple of kGroup (host checks)
    issue_group(0);
    int mine = (lane < min(kWave, a.T)) ? ip[lane] : 0;       // first 64 fine indices, entry i in lane i

    bf16x8 bq[2];
    {
        const bf16* qp = (const bf16*)a.qr + ((int64_t)bh * N1 + g) * kTile + lane * 8;
        bq[0] = ld16(qp);       // 1/sqrt(64) is a power of two: scaling q before the product (as the
        bq[1] = ld16(qp + 512); // reference does) equals scaling the fp32 scores, done in the exponent
    }
    SoftmaxState st;
    init_state(st);

    KvRegs ra, rb;

    // ---- shared blocks, out of LDS.  The barrier at the top of round grp says two things: every
    // wave's part of group grp has landed, and every wave is done reading the other buffer
    // (group grp - 1), which the next fetch overwrites.
    float w_prev = 1.f;
    for (int grp = 0; grp < n_groups; grp++) {
        wait_vm0();
        __syncthreads();
        // weight(previous segment) / weight(this one); nothing is accumulated before group 0
        const float w_here = a.lvl[shared_level(a.lvl, a.levels, kGroup * grp)].w;
        if (grp > 0 && w_here != w_prev) rescale(st, w_prev / w_here);
        w_prev = w_here;
        // (LDS reads first: the compiler makes every LDS read wait for all copies into LDS that
        // were issued before it, which would serialise the next fetch with the arithmetic of this group)
        load_step_lds(ra, &sh[grp & 1][0][0], lane);
        load_step_lds(rb, &sh[grp & 1][NB][0], lane);
        if (grp + 1 < n_groups) issue_group(grp + 1);
        if (grp == 0) start_reference(st, bq, ra);
        compute_step(st, bq, ra);
        compute_step(st, bq, rb);
    }
    rescale(st, w_prev);                                      // fine tokens weigh 1

    wait_all_mem();     // nothing is in flight here: said for the compiler (see wait_all_mem)
    // ---- fine blocks, private to the wave.  Their indices are fetched 64 at a time, entry i into
    // lane i, and handed out with readlane (a copy into LDS counts as a store for the compiler,
    // after which it no longer turns uniform loads into scalar loads; a vector load inside the
    // pipelined loop would wait for every tile load issued before it).
    for (int c0 = 0; c0 < a.T; c0 += kWave) {
        const int cn = min(kWave, a.T - c0);                  // a multiple of 4: an even number of steps
        if (c0 > 0) mine = (lane < cn) ? ip[c0 + lane] : 0;
        const int n_fine = cn / NB;
        auto describe = [=](int t, StepDesc& d) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < NB; j++) {
                const int blk = clampi(__builtin_amdgcn_readlane(mine, NB * t + j), 0, N1 - 1);
                d.kb[j] = kr + (int64_t)blk * kTile;
                d.vtb[j] = vt + (int64_t)blk * kTile;
            }
        };
        // The prefetch is unconditional (past the end it re-reads the last step) so that the loop
        // body is straight-line code: with the loads inside a branch the compiler has to drain the
        // memory queue (s_waitcnt vmcnt(0)) before every step and the overlap is lost.
        StepDesc d;
        describe(0, d);
        load_step(ra, d, lane);
        for (int t = 0; t < n_fine; t += 2) {
            describe(min(t + 1, n_fine - 1), d);
            load_step(rb, d, lane);
            compute_step(st, bq, ra);
            if (t + 1 >= n_fine) break;
            describe(min(t + 2, n_fine - 1), d);
            load_step(ra, d, lane);
            compute_step(st, bq, rb);
        }
    }

    finish_query_block(a, st, bh, b, h, g, lane);
}

// ---------------------------------------------------------------------------------------
// Two sibling query blocks per wave (topk <= 32).  Both walk the same pooled blocks, and on coherent inputs most
// of their fine blocks coincide, so every operand tile that both need is fetched once and multiplied twice: the
// wave first sorts the two fine lists into [blocks both selected | only the first | only the second] and walks
// that list in steps of NB blocks, a step of the first part feeding both soft-max states.  What bounds these
// kernels is the rate at which tiles arrive from the L2, and this removes a quarter to a half of them.
// A row that names a block twice keeps the plain walk (nothing is shared).
// ---------------------------------------------------------------------------------------

__global__ __launch_bounds__(256, 3) void attn_fwd_pair_kernel(llsa_attn_fwd_args a) {
    static_assert(NB == 2 && kGroup == 4, "the shared phase reads an LDS buffer of four blocks as two steps of two");
    __shared__ __align__(16) bf16 sh[2][kGroup][2 * kTile];
    __shared__ int order[4][kWave];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int N1 = a.N / kBlk, T = a.T;
    const int lid = xcd_logical_id();
    const int g = (lid % (int)gridDim.x) * 8 + 2 * wave;      // query blocks g and g + 1 (the host checks N1 % 8 == 0)
    const int bh = lid / (int)gridDim.x, b = bh / a.H, h = bh % a.H;

    const bf16* kr = (const bf16*)a.kr + (int64_t)bh * N1 * kTile;
    const bf16* vt = (const bf16*)a.vt + (int64_t)bh * N1 * kTile;
    const int* ip = a.idx + ((int64_t)bh * N1 + g) * T;

    SharedList sl = shared_list(a.lvl, a.levels, a.N, bh, g, lane);
    bf16* const sh0 = &sh[0][0][0];
    auto issue_group = [&](int grp) __attribute__((always_inline)) {
        const SharedBlock sb = shared_block(sl, a.lvl, a.levels, a.N, bh, kGroup * grp + wave);
        const bf16* kb = (const bf16*)a.lvl[sb.level].kr + sb.tile;
        const bf16* vb = (const bf16*)a.lvl[sb.level].vt + sb.tile;
        bf16* dst = sh0 + ((grp & 1) * kGroup + wave) * (2 * kTile);
        copy16_global_to_lds(kb + lane * 8, dst);
        copy16_global_to_lds(kb + 512 + lane * 8, dst + 512);
        copy16_global_to_lds(vb + lane * 8, dst + kTile);
        copy16_global_to_lds(vb + 512 + lane * 8, dst + kTile + 512);
    };
    const int n_groups = sl.n_blocks / kGroup;
    issue_group(0);

    // ---- the two fine lists, sorted into [both | only the first | only the second]; entry i ends in lane i
    const PairOrder po = pair_order(ip, T, N1, lane, order[wave]);
    const int mine = po.mine;
    const int steps_both = po.n_both / NB, steps_only = (T - po.n_both) / NB, n_steps = steps_both + 2 * steps_only;

    bf16x8 bq[2][2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const bf16* qp = (const bf16*)a.qr + ((int64_t)bh * N1 + g + u) * kTile + lane * 8;
        bq[u][0] = ld16(qp);
        bq[u][1] = ld16(qp + 512);
    }
    SoftmaxState st[2];
    init_state(st[0]);
    init_state(st[1]);
    KvRegs ra, rb;

    float w_prev = 1.f;
    for (int grp = 0; grp < n_groups; grp++) {
        wait_vm0();
        __syncthreads();
        const float w_here = a.lvl[shared_level(a.lvl, a.levels, kGroup * grp)].w;
        if (grp > 0 && w_here != w_prev) {
            rescale(st[0], w_prev / w_here);
            rescale(st[1], w_prev / w_here);
        }
        w_prev = w_here;
        load_step_lds(ra, &sh[grp & 1][0][0], lane);
        load_step_lds(rb, &sh[grp & 1][NB][0], lane);
        if (grp + 1 < n_groups) issue_group(grp + 1);
        if (grp == 0) {
            start_reference(st[0], bq[0], ra);
            start_reference(st[1], bq[1], ra);
        }
        compute_step2(st[0], st[1], bq[0], bq[1], ra);
        compute_step2(st[0], st[1], bq[0], bq[1], rb);
    }
    rescale(st[0], w_prev);                                   // fine tokens weigh 1
    rescale(st[1], w_prev);
    wait_all_mem();

    auto describe = [=](int t, StepDesc& d) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < NB; j++) {
            const int blk = __builtin_amdgcn_readlane(mine, NB * t + j);
            d.kb[j] = kr + (int64_t)blk * kTile;
            d.vtb[j] = vt + (int64_t)blk * kTile;
        }
    };
    auto work = [&](int t, const KvRegs& regs) __attribute__((always_inline)) {
        if (t < steps_both) compute_step2(st[0], st[1], bq[0], bq[1], regs);
        else if (t < steps_both + steps_only) compute_step(st[0], bq[0], regs);
        else compute_step(st[1], bq[1], regs);
    };
    StepDesc d;
    describe(0, d);
    load_step(ra, d, lane);
    for (int t = 0; t < n_steps; t += 2) {
        describe(min(t + 1, n_steps - 1), d);
        load_step(rb, d, lane);
        work(t, ra);
        if (t + 1 >= n_steps) break;
        describe(min(t + 2, n_steps - 1), d);
        load_step(ra, d, lane);
        work(t + 1, rb);
    }
    finish_query_block(a, st[0], bh, b, h, g, lane);
    finish_query_block(a, st[1], bh, b, h, g + 1, lane);
}

}  // namespace llsa

using namespace llsa;

extern "C" int llsa_attn_fwd(const llsa_attn_fwd_args* a, void* stream) {
    LLSA_REQUIRE(a != nullptr, "attn_fwd: null args");
    LLSA_REQUIRE(a->levels >= 1 && a->levels <= LLSA_MAX_LEVELS, "attn_fwd: levels must be 1..%d", LLSA_MAX_LEVELS);
    LLSA_REQUIRE(a->B > 0 && a->H > 0 && a->N > 0, "attn_fwd: bad B/H/N");
    LLSA_REQUIRE(a->qr && a->kr && a->vt && a->idx && a->o && a->lse, "attn_fwd: null tensor");
    LLSA_REQUIRE(a->T >= 4 && a->T % 4 == 0 && a->T <= a->N / 16, "attn_fwd: topk=%d must be a multiple of 4 and <= N/16", a->T);
    const int64_t mult = coarsest_multiple(a->levels);
    LLSA_REQUIRE(a->N % mult == 0,
                 "attn_fwd: %d level(s) need N %% %lld == 0 (N=%d): the coarsest level is walked in 64-token tiles of its N/16^levels pooled tokens",
                 a->levels, (long long)mult, a->N);
    int listed = 0;
    int64_t span = 256;                                       // tokens under one block of level l
    for (int l = 1; l <= a->levels; l++, span *= 16) {
        const llsa_fwd_level& lv = a->lvl[l - 1];
        LLSA_REQUIRE(lv.kr && lv.vt && aligned16(lv.kr) && aligned16(lv.vt), "attn_fwd: tiles of level %d missing or not 16-byte aligned", l);
        LLSA_REQUIRE(lv.w > 0.f, "attn_fwd: the weight of level %d must be > 0", l);
        if (l < a->levels) {
            LLSA_REQUIRE(lv.sel != nullptr, "attn_fwd: selection of level %d missing", l);
            LLSA_REQUIRE(lv.T >= 4 && lv.T % 4 == 0 && lv.T <= a->N / span, "attn_fwd: topk of level %d (%d) must be a multiple of 4 and <= N/%lld",
                         l, lv.T, (long long)span);
            listed += lv.T;
        }
    }
    LLSA_REQUIRE(listed <= LLSA_POOLED_TOPK_MAX, "attn_fwd: the topk of the pooled levels together (%d) must not exceed %d", listed,
                 LLSA_POOLED_TOPK_MAX);
    LLSA_REQUIRE(aligned16(a->qr) && aligned16(a->kr) && aligned16(a->vt) && aligned16(a->o), "attn_fwd: tensors must be 16-byte aligned");
    LLSA_REQUIRE((a->sob % 4 == 0) && (a->soh % 4 == 0) && (a->son % 4 == 0), "attn_fwd: rows of o must be 8-byte aligned");
    const int N1 = a->N / 16;
    if (a->T <= kPairMaxTopk && N1 % 8 == 0)
        hipLaunchKernelGGL(attn_fwd_pair_kernel, dim3(N1 / 8, a->B * a->H), dim3(256), 0, (hipStream_t)stream, *a);
    else
        hipLaunchKernelGGL(attn_fwd_kernel, dim3((N1 + 3) / 4, a->B * a->H), dim3(256), 0, (hipStream_t)stream, *a);
    return launch_status("attn_fwd");
}
