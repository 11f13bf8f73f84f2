// Block selection: dense coarsest-level top-k and parent-guided fine top-k.
//
// The kernels score one tile of 16 pooled queries against 16-key tiles with the bf16 MFMA,
// park the scores of the 16 rows in LDS and then let each wave select the T best entries of
// "its" rows: by radix selection when a row fits in LDS, by repeated wave-wide arg-max over
// chunks otherwise.  The order is total -- higher score first, equal scores by smaller key
// index -- so the result does not depend on how the work is split.
#include "llsa_device.h"
#include "llsa_host.h"
#include "../../include/llsa_hip.h"

namespace llsa {

constexpr int kMaxT = 64;        // largest supported top-k
constexpr int kChunk = 512;      // keys scored per pass of the dense kernel
constexpr int kMaxCand = 512;    // candidates per parent in the sparse kernel (T2 * 16)
constexpr int kNoIdx = 0x7fffffff;

// Removes the T best entries of `row[0..npos)` (a wave's private LDS row) one by one.
// Lane `lane` only ever touches positions congruent to it mod 64, so no barrier is
// needed between iterations.  Taken entries are overwritten with NaN, which never
// compares greater or equal.  Winners are written by lane 0.
template <typename IdxFn>
__device__ __forceinline__ void wave_topk_row(float* row, int npos, int T, IdxFn gidx_of, float* win_val,
                                              int* win_idx) {
    const int lane = threadIdx.x & (kWave - 1);
    for (int t = 0; t < T; t++) {
        float bv = -INFINITY;
        int bi = kNoIdx, bp = -1;
        for (int pos = lane; pos < npos; pos += kWave) {
            const float v = row[pos];
            const int gi = gidx_of(pos);
            if (v > bv || (v == bv && gi < bi)) {
                bv = v;
                bi = gi;
                bp = pos;
            }
        }
        float wv = bv;
        int wi = bi;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const float ov = __shfl_xor(wv, off);
            const int oi = __shfl_xor(wi, off);
            if (ov > wv || (ov == wv && oi < wi)) {
                wv = ov;
                wi = oi;
            }
        }
        if (bp >= 0 && bi == wi && bv == wv) row[bp] = __builtin_nanf("");
        if (lane == 0) {
            win_val[t] = (wi == kNoIdx) ? __builtin_nanf("") : wv;
            win_idx[t] = wi;
        }
    }
}

// S^T tile: rows = 16 keys starting at krow, columns = the wave's 16 queries (bq).
// Lane l gets the scores of query l%16 against keys 4*(l/16) .. +3 of the tile.
__device__ __forceinline__ f32x4 score_tile(const bf16* krow, const bf16x8 bq[2]) {
    const int lane = threadIdx.x & (kWave - 1);
    const bf16* p = krow + (lane & 15) * kD + (lane >> 4) * 8;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    acc = mfma_bf16(ld16(p), bq[0], acc);
    acc = mfma_bf16(ld16(p + 32), bq[1], acc);
    return acc;
}

__global__ __launch_bounds__(256) void topk_dense_kernel(const bf16* __restrict__ pq, const bf16* __restrict__ pk,
                                                         int* __restrict__ out, int n, int T, int round_scores) {
    __shared__ float sc[16][kMaxT + kChunk + 1];
    __shared__ int carry_idx[16][kMaxT];
    __shared__ float win_val[16][kMaxT];
    __shared__ int win_idx[16][kMaxT];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bh = blockIdx.y, q0 = blockIdx.x * 16;
    const bf16* pqb = pq + ((int64_t)bh * n + q0) * kD;
    const bf16* pkb = pk + (int64_t)bh * n * kD;

    bf16x8 bq[2];
    bq[0] = ld16(pqb + (lane & 15) * kD + (lane >> 4) * 8);
    bq[1] = ld16(pqb + (lane & 15) * kD + (lane >> 4) * 8 + 32);

    for (int i = tid; i < 16 * T; i += 256) {
        sc[i / T][i % T] = __builtin_nanf("");
        carry_idx[i / T][i % T] = kNoIdx;
    }
    __syncthreads();

    for (int base = 0; base < n; base += kChunk) {
        const int len = min(kChunk, n - base);
        for (int tile = wave; tile < len / 16; tile += 4) {
            f32x4 s = score_tile(pkb + (int64_t)(base + tile * 16) * kD, bq);
#pragma unroll
            for (int e = 0; e < 4; e++)
                sc[lane & 15][T + tile * 16 + 4 * (lane >> 4) + e] = round_scores ? rn_bf16(s[e]) : s[e];
        }
        __syncthreads();
        for (int row = wave; row < 16; row += 4) {
            const int* ci = carry_idx[row];
            wave_topk_row(
                sc[row], T + len, T, [=](int pos) { return pos < T ? ci[pos] : base + pos - T; }, win_val[row],
                win_idx[row]);
        }
        __syncthreads();
        for (int i = tid; i < 16 * T; i += 256) {
            sc[i / T][i % T] = win_val[i / T][i % T];
            carry_idx[i / T][i % T] = win_idx[i / T][i % T];
        }
        __syncthreads();
    }
    for (int i = tid; i < 16 * T; i += 256) out[((int64_t)bh * n + q0 + i / T) * T + i % T] = win_idx[i / T][i % T];
}

// ---------------------------------------------------------------------------------------
// Radix selection.  Scores are mapped to unsigned integers that sort like the floats; the
// T-th largest is found one bit at a time from the top with a wave-wide count per bit
// (a compare, a ballot and a scalar popcount per entry, no cross-lane data movement), then
// everything above it -- plus as many entries equal to it as are still needed, smallest
// index first -- is compacted and put in final order by rank counting among the T winners.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ unsigned ordered_bits(float f) {
    if (f != f) return 0u;                                    // NaN sorts below everything
    const unsigned b = __float_as_uint(f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// u[0..npos): ordered scores of one row (LDS); gidx_of(pos): global index of a position.
// Each lane keeps its E entries (positions lane, lane + 64, ...) in registers, so a bit step is
// E compares + ballots + scalar popcounts with no memory access.
// sel_u / sel_i: 64 entries of LDS scratch each.  out[0..T): result, global memory.
// low_bit: the keys' bits below it are known to be zero (16 for scores rounded to bf16) and are not
// looked at; idx_bits: the global indices are below 2^idx_bits (the tie pass starts there).
template <int E, typename IdxFn>
__device__ __forceinline__ void wave_topk_radix(const unsigned* u, int npos, int T, IdxFn gidx_of, unsigned* sel_u,
                                                int* sel_i, int* out, int lane, int low_bit, int idx_bits) {
    unsigned uk[E];
    unsigned gk[E];
    bool ok[E];
#pragma unroll
    for (int e = 0; e < E; e++) {
        const int pos = lane + e * kWave;
        ok[e] = pos < npos;
        uk[e] = ok[e] ? u[pos] : 0u;
        gk[e] = ok[e] ? (unsigned)gidx_of(pos) : 0xFFFFFFFFu;
    }
    // Invalid slots hold key 0 and never equal `want` (its current bit is set), so the bit loop
    // needs no validity mask.  `match` counts the entries that agree with the decided bits; once
    // it equals the number still to take, all of them are winners and the remaining bits need
    // not be looked at (tau = prefix with zero low bits then selects exactly those).
    unsigned prefix = 0;
    int remaining = T, match = npos;
    for (int bit = 31; bit >= low_bit && match != remaining; bit--) {
        const unsigned msk = (bit == 31) ? 0x80000000u : ((0xFFFFFFFFu << (bit + 1)) | (1u << bit));
        const unsigned want = prefix | (1u << bit);
        int cnt1 = 0;
#pragma unroll
        for (int e = 0; e < E; e++) cnt1 += __popcll(__ballot((uk[e] & msk) == want));
        if (cnt1 >= remaining) {
            prefix = want;
            match = cnt1;
        } else {
            remaining -= cnt1;
            match -= cnt1;
        }
    }
    const unsigned tau = prefix;                              // the T-th largest score
    int n_eq = 0;
#pragma unroll
    for (int e = 0; e < E; e++) n_eq += __popcll(__ballot(ok[e] && uk[e] == tau));
    unsigned idx_thr = 0xFFFFFFFFu;
    if (n_eq > remaining) {                                   // ties at the threshold: keep the smallest indices
        unsigned p2 = 0;
        int rem2 = remaining;
        for (int bit = idx_bits - 1; bit >= 0; bit--) {
            const unsigned msk = (0xFFFFFFFFu << (bit + 1)) | (1u << bit);
            int cnt0 = 0;
#pragma unroll
            for (int e = 0; e < E; e++) cnt0 += __popcll(__ballot(ok[e] && uk[e] == tau && (gk[e] & msk) == p2));
            if (cnt0 < rem2) {
                rem2 -= cnt0;
                p2 |= (1u << bit);
            }
        }
        idx_thr = p2;
    }
    if (lane < T) {
        sel_u[lane] = 0u;
        sel_i[lane] = kNoIdx;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    int base_slot = 0;
#pragma unroll
    for (int e = 0; e < E; e++) {
        const bool sel = ok[e] && (uk[e] > tau || (uk[e] == tau && gk[e] <= idx_thr));
        const unsigned long long m = __ballot(sel);
        const int slot = base_slot + __popcll(m & ((1ull << lane) - 1ull));
        if (sel && slot < T) {
            sel_u[slot] = uk[e];
            sel_i[slot] = (int)gk[e];
        }
        base_slot += __popcll(m);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    {   // final order by rank counting among the T winners: winner j sits in lane j and is handed round with readlane
        const unsigned mu = sel_u[lane];
        const int mi = sel_i[lane];
        int rank = 0;
        for (int j = 0; j < T; j++) {
            const unsigned ou = (unsigned)__builtin_amdgcn_readlane((int)mu, j);
            const int oi = __builtin_amdgcn_readlane(mi, j);
            rank += (ou > mu || (ou == mu && (oi < mi || (oi == mi && j < lane)))) ? 1 : 0;
        }
        if (lane < T) out[rank] = mi;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// entries per lane as a compile-time bound: 1, 2, 4, 8 or 16
template <typename IdxFn>
__device__ __forceinline__ void wave_topk_radix_any(const unsigned* u, int npos, int T, IdxFn gidx_of, unsigned* sel_u,
                                                    int* sel_i, int* out, int lane, int low_bit, int idx_bits) {
    if (npos <= 64) wave_topk_radix<1>(u, npos, T, gidx_of, sel_u, sel_i, out, lane, low_bit, idx_bits);
    else if (npos <= 128) wave_topk_radix<2>(u, npos, T, gidx_of, sel_u, sel_i, out, lane, low_bit, idx_bits);
    else if (npos <= 256) wave_topk_radix<4>(u, npos, T, gidx_of, sel_u, sel_i, out, lane, low_bit, idx_bits);
    else if (npos <= 512) wave_topk_radix<8>(u, npos, T, gidx_of, sel_u, sel_i, out, lane, low_bit, idx_bits);
    else wave_topk_radix<16>(u, npos, T, gidx_of, sel_u, sel_i, out, lane, low_bit, idx_bits);
}

constexpr int kRadixMaxN = 1024;      // keys per row the radix kernels keep in LDS

// dense selection for n <= kRadixMaxN: 16 query rows per workgroup, all n keys scored into LDS
// (16 waves: one row each, so the 16 selections run side by side instead of four deep)
__global__ __launch_bounds__(1024) void topk_dense_radix_kernel(const bf16* __restrict__ pq, const bf16* __restrict__ pk,
                                                                int* __restrict__ out, int n, int T, int round_scores) {
    HIP_DYNAMIC_SHARED(unsigned, su)                          // [16][n + 1]
    __shared__ unsigned sel_u[16][kWave];
    __shared__ int sel_i[16][kWave];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bh = blockIdx.y, q0 = blockIdx.x * 16;
    const int stride = n + 1;
    const bf16* pqb = pq + ((int64_t)bh * n + q0) * kD;
    const bf16* pkb = pk + (int64_t)bh * n * kD;
    bf16x8 bq[2];
    bq[0] = ld16(pqb + (lane & 15) * kD + (lane >> 4) * 8);
    bq[1] = ld16(pqb + (lane & 15) * kD + (lane >> 4) * 8 + 32);
    for (int tile = wave; tile < n / 16; tile += 16) {
        f32x4 s = score_tile(pkb + (int64_t)tile * 16 * kD, bq);
#pragma unroll
        for (int e = 0; e < 4; e++)
            // (a score rounded to bf16 has 16 constant low key bits -- ones when negative; cleared, the
            // selection below need not look at them)
            su[(lane & 15) * stride + tile * 16 + 4 * (lane >> 4) + e] =
                round_scores ? (ordered_bits(rn_bf16(s[e])) & 0xFFFF0000u) : ordered_bits(s[e]);
    }
    __syncthreads();
    for (int row = wave; row < 16; row += 16)
        wave_topk_radix_any(
            su + row * stride, n, T, [](int pos) { return pos; }, sel_u[wave], sel_i[wave],
            out + ((int64_t)bh * n + q0 + row) * T, lane, round_scores ? 16 : 0, 32 - __builtin_clz(n - 1));
}

constexpr int kSparseWaves = 8;       // two rows per wave: four workgroups fit a CU and the grid is one round
// pq_par != nullptr: the parents are selected here first -- row G of the level above (N1/16 tokens, at most
// kCascadeMaxParents) against all of its keys, scores rounded to bf16, top T2 as topk_dense_radix_kernel does it -- and
// written to par_out; otherwise they are read from pidx.
__global__ __launch_bounds__(64 * kSparseWaves) void topk_sparse_kernel(const bf16* __restrict__ pq, const bf16* __restrict__ pk,
                                                           const int* __restrict__ pidx, int* __restrict__ out, int N1,
                                                           int T, int T2, const bf16* __restrict__ pq_par,
                                                           const bf16* __restrict__ pk_par, int* __restrict__ par_out) {
    __shared__ unsigned su[16][kMaxCand + 1];
    __shared__ int cand[kMaxCand];
    __shared__ unsigned sel_u[16][kWave];
    __shared__ int sel_i[16][kWave];
    __shared__ int par[kMaxCand / 16];
    static_assert(16 * (kMaxCand + 1) >= kRadixMaxN, "the parents' scores borrow the candidates' score rows");

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bh = blockIdx.y, G = blockIdx.x;
    const int N2 = N1 / kBlk, C = T2 * kBlk;
    const bf16* pqb = pq + ((int64_t)bh * N1 + G * kBlk) * kD;
    const bf16* pkb = pk + (int64_t)bh * N1 * kD;

    if (pq_par != nullptr) {
        unsigned* su_par = &su[0][0];
        const bf16* qt = pq_par + ((int64_t)bh * N2 + (G & ~15)) * kD;     // the tile of 16 rows that holds row G
        bf16x8 bp[2];
        bp[0] = ld16(qt + (lane & 15) * kD + (lane >> 4) * 8);
        bp[1] = ld16(qt + (lane & 15) * kD + (lane >> 4) * 8 + 32);
        for (int tile = wave; tile < N2 / 16; tile += kSparseWaves) {
            f32x4 s = score_tile(pk_par + ((int64_t)bh * N2 + tile * 16) * kD, bp);
            if ((lane & 15) == (G & 15)) {
#pragma unroll
                for (int e = 0; e < 4; e++) su_par[tile * 16 + 4 * (lane >> 4) + e] = ordered_bits(rn_bf16(s[e])) & 0xFFFF0000u;
            }
        }
        __syncthreads();
        if (wave == 0)
            wave_topk_radix_any(
                su_par, N2, T2, [](int pos) { return pos; }, sel_u[0], sel_i[0], par, lane, 16, 32 - __builtin_clz(N2 - 1));
        __syncthreads();
        if (tid < T2) par_out[((int64_t)bh * N2 + G) * T2 + tid] = par[tid];
    } else {
        if (tid < T2) par[tid] = clampi(pidx[((int64_t)bh * N2 + G) * T2 + tid], 0, N2 - 1);
        __syncthreads();
    }
    for (int i = tid; i < C; i += 64 * kSparseWaves) cand[i] = par[i / kBlk] * kBlk + (i % kBlk);
    bf16x8 bq[2];
    bq[0] = ld16(pqb + (lane & 15) * kD + (lane >> 4) * 8);
    bq[1] = ld16(pqb + (lane & 15) * kD + (lane >> 4) * 8 + 32);
    __syncthreads();

    for (int a = wave; a < T2; a += kSparseWaves) {
        f32x4 s = score_tile(pkb + (int64_t)cand[a * kBlk] * kD, bq);
#pragma unroll
        for (int e = 0; e < 4; e++) su[lane & 15][a * kBlk + 4 * (lane >> 4) + e] = ordered_bits(s[e]);
    }
    __syncthreads();
    for (int row = wave; row < 16; row += kSparseWaves)
        wave_topk_radix_any(
            su[row], C, T, [&](int pos) { return cand[pos]; }, sel_u[wave], sel_i[wave],
            out + ((int64_t)bh * N1 + G * kBlk + row) * T, lane, 0, 32 - __builtin_clz(N1 - 1));
}

}  // namespace llsa

using namespace llsa;

extern "C" int llsa_topk_dense(const void* pq, const void* pk, int32_t* out_idx, int B, int H, int n, int T,
                               int round_scores, void* stream) {
    LLSA_REQUIRE(pq && pk && out_idx, "topk_dense: null argument");
    LLSA_REQUIRE(B > 0 && H > 0 && n > 0 && n % 16 == 0, "topk_dense: n=%d must be a positive multiple of 16", n);
    LLSA_REQUIRE(T >= 1 && T <= kMaxT && T <= n, "topk_dense: need 1 <= T <= min(%d, n=%d), got %d", kMaxT, n, T);
    LLSA_REQUIRE(aligned16(pq) && aligned16(pk), "topk_dense: inputs must be 16-byte aligned");
    if (n <= kRadixMaxN) {
        const int lds = (int)sizeof(unsigned) * 16 * (n + 1);
        if (lds > 60 * 1024) {
            hipError_t e = hipFuncSetAttribute((const void*)topk_dense_radix_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
            if (e != hipSuccess) return fail(-101, "topk_dense: cannot raise dynamic LDS to %d bytes: %s", lds, hipGetErrorString(e));
        }
        hipLaunchKernelGGL(topk_dense_radix_kernel, dim3(n / 16, B * H), dim3(1024), sizeof(unsigned) * 16 * (n + 1),
                           (hipStream_t)stream, (const bf16*)pq, (const bf16*)pk, out_idx, n, T, round_scores);
    } else
        hipLaunchKernelGGL(topk_dense_kernel, dim3(n / 16, B * H), dim3(256), 0, (hipStream_t)stream, (const bf16*)pq,
                           (const bf16*)pk, out_idx, n, T, round_scores);
    return launch_status("topk_dense");
}

extern "C" int llsa_topk_sparse(const void* pq, const void* pk, const int32_t* parent_idx, int32_t* out_idx, int B, int H,
                                int N1, int T, int T2, void* stream) {
    LLSA_REQUIRE(pq && pk && parent_idx && out_idx, "topk_sparse: null argument");
    LLSA_REQUIRE(B > 0 && H > 0 && N1 > 0 && N1 % 16 == 0, "topk_sparse: N1=%d must be a positive multiple of 16", N1);
    LLSA_REQUIRE(T2 >= 1 && T2 * 16 <= kMaxCand && T2 <= N1 / 16, "topk_sparse: need 1 <= T2 <= min(%d, N1/16), got %d", kMaxCand / 16, T2);
    LLSA_REQUIRE(T >= 1 && T <= kMaxT && T <= T2 * 16, "topk_sparse: need 1 <= T <= min(%d, 16*T2), got %d", kMaxT, T);
    LLSA_REQUIRE(aligned16(pq) && aligned16(pk), "topk_sparse: inputs must be 16-byte aligned");
    hipLaunchKernelGGL(topk_sparse_kernel, dim3(N1 / 16, B * H), dim3(64 * kSparseWaves), 0, (hipStream_t)stream, (const bf16*)pq,
                       (const bf16*)pk, parent_idx, out_idx, N1, T, T2, (const bf16*)nullptr, (const bf16*)nullptr, (int*)nullptr);
    return launch_status("topk_sparse");
}

// (a workgroup selects its parent row on one wave: beyond a few hundred parent tokens the separate dense kernel,
// sixteen rows per workgroup side by side, is faster -- 277 vs 120 + 43 us at 1024)
constexpr int kCascadeMaxParents = 256;
extern "C" int llsa_topk_cascade_max_parents(void) { return kCascadeMaxParents; }

extern "C" int llsa_topk_cascade(const void* pq_parent, const void* pk_parent, int32_t* parent_out, const void* pq, const void* pk,
                                 int32_t* out_idx, int B, int H, int N1, int T, int T2, void* stream) {
    LLSA_REQUIRE(pq_parent && pk_parent && parent_out && pq && pk && out_idx, "topk_cascade: null argument");
    LLSA_REQUIRE(B > 0 && H > 0 && N1 > 0 && N1 % 256 == 0, "topk_cascade: N1=%d must be a positive multiple of 256", N1);
    LLSA_REQUIRE(N1 / 16 <= kCascadeMaxParents, "topk_cascade: at most %d parent tokens (got %d): use llsa_topk_dense and llsa_topk_sparse",
                 kCascadeMaxParents, N1 / 16);
    LLSA_REQUIRE(T2 >= 1 && T2 * 16 <= kMaxCand && T2 <= N1 / 16, "topk_cascade: need 1 <= T2 <= min(%d, N1/16), got %d", kMaxCand / 16, T2);
    LLSA_REQUIRE(T >= 1 && T <= kMaxT && T <= T2 * 16, "topk_cascade: need 1 <= T <= min(%d, 16*T2), got %d", kMaxT, T);
    LLSA_REQUIRE(aligned16(pq) && aligned16(pk) && aligned16(pq_parent) && aligned16(pk_parent), "topk_cascade: inputs must be 16-byte aligned");
    hipLaunchKernelGGL(topk_sparse_kernel, dim3(N1 / 16, B * H), dim3(64 * kSparseWaves), 0, (hipStream_t)stream, (const bf16*)pq,
                       (const bf16*)pk, (const int*)nullptr, out_idx, N1, T, T2, (const bf16*)pq_parent, (const bf16*)pk_parent, parent_out);
    return launch_status("topk_cascade");
}
