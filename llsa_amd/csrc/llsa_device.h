// Device-side building blocks shared by the gfx950 kernels: vector types, the bf16
// 16x16x32 MFMA wrapper with its register layout, 64-lane reductions, bf16 rounding.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace llsa {

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;

constexpr int kWave = 64;        // CDNA wavefront
constexpr int kBlk = 16;         // tokens per block (block_size of the operator)
constexpr int kD = 64;           // head dimension the MFMA kernels are specialised for
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kScale = 0.125f;                          // 1/sqrt(kD)
constexpr float kScaleLog2e = 0.125f * 1.4426950408889634f;

// v_mfma_f32_16x16x32_bf16:  D(16x16) = A(16x32) * B(32x16) + C.
//   lane l supplies  A[row = l%16][k = 8*(l/16) + e]   e = 0..7
//                    B[k = 8*(l/16) + e][col = l%16]
//   and owns         D[row = 4*(l/16) + e][col = l%16] e = 0..3
// Both operands are "8 consecutive k for one row/column", i.e. a 16-byte load from a
// row-major matrix whose fast axis is the contraction axis.
__device__ __forceinline__ f32x4 mfma_bf16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 ld16(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x4 ld8(const bf16* p) { return *reinterpret_cast<const bf16x4*>(p); }
__device__ __forceinline__ void st16(bf16* p, bf16x8 v) { *reinterpret_cast<bf16x8*>(p) = v; }
__device__ __forceinline__ void st8(bf16* p, bf16x4 v) { *reinterpret_cast<bf16x4*>(p) = v; }

__device__ __forceinline__ bf16x8 cat(bf16x4 lo, bf16x4 hi) {
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}
__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; i++) z[i] = (bf16)0.0f;
    return z;
}
__device__ __forceinline__ bf16x4 zero4() {
    bf16x4 z;
#pragma unroll
    for (int i = 0; i < 4; i++) z[i] = (bf16)0.0f;
    return z;
}
__device__ __forceinline__ bf16x4 cvt4(f32x4 v) {
    bf16x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = (bf16)v[i];
    return r;
}

// round-to-nearest-even through bf16, value kept in fp32
__device__ __forceinline__ float rn_bf16(float x) { return (float)(bf16)x; }

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// Reductions over the four lanes {l, l^16, l^32, l^48} that share one MFMA column, with the lane
// swaps of gfx950 (v_permlane16_swap, v_permlane32_swap: vector-ALU instructions, where a shuffle
// goes through the LDS unit and makes the wave wait for it).  swap16(v, v) leaves in its two
// results v of this lane and v of lane l^16 (which is which depends on the row), swap32 the same
// for l^32; both reductions are symmetric, so every lane of the four ends with the same bits.
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
__device__ __forceinline__ float quad_max(float v) {
    u32x2 a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    u32x2 b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_sum(float v) {
    u32x2 a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    u32x2 b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Operand tiles.  The attention kernels never read K/V/Q/dO row-major: a 16-row x 64-channel
// block (1024 bf16 = 2 KB) is stored twice, each time in exactly the order the 64 lanes of a
// wave consume it as an MFMA operand, so that every operand load is one fully coalesced
// instruction (lane l reads bytes [16 l, 16 l + 16) or [8 l, 8 l + 8) of a contiguous piece)
// instead of 64 scattered 16-byte accesses, which would saturate the L1's access rate.
//   R tile ("rows", contraction over channels):  element (row i, channel c) at
//        ((c >> 3) * 16 + i) * 8 + (c & 7)
//     lane l, step s (channels 32 s ..) loads 8 elements at  s * 512 + l * 8
//   T tile ("tokens", contraction over the 16 rows): element (row t, channel c) at
//        (((c >> 4) * 4 + (t >> 2)) * 16 + (c & 15)) * 4 + (t & 3)
//     lane l, channel tile dt (channels 16 dt ..) loads 4 elements at  dt * 256 + l * 4
constexpr int kTile = kBlk * kD;     // elements per block tile
__device__ __forceinline__ int r_tile_off(int i, int c) { return ((c >> 3) * 16 + i) * 8 + (c & 7); }
__device__ __forceinline__ int t_tile_off(int t, int c) { return (((c >> 4) * 4 + (t >> 2)) * 16 + (c & 15)) * 4 + (t & 3); }

// A T operand out of an R tile that sits in LDS, with the transposing LDS read of gfx950
// (ds_read_b64_tr_b16).  Within each group of 16 lanes, lane j supplies the address of four
// consecutive 16-bit elements and lane i receives element i%4 of the chunks supplied by lanes
// i/4, 4 + i/4, 8 + i/4, 12 + i/4.  Pointing lane j at (token 4*(l/16) + j/4, channels
// 16*dt + 4*(j%4) ..+3) therefore hands lane i tokens 4*(l/16)..+3 of channel 16*dt + i: the T
// operand.  So K/Q/dO are fetched from HBM once, as R tiles, and the second orientation is
// made on chip instead of being read from a second copy.
typedef __attribute__((ext_vector_type(4))) short s16x4;
__device__ __forceinline__ bf16x4 lds_t_operand(const bf16* r_tile_in_lds, int dt, int lane) {
    const int j = lane & 15, q = lane >> 4;
    const bf16* p = r_tile_in_lds + r_tile_off(4 * q + (j >> 2), 16 * dt + 4 * (j & 3));
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
    return __builtin_bit_cast(bf16x4, v);
}

// Asynchronous 16-byte-per-lane copy from global memory straight into LDS (no registers):
// lane l's 16 bytes land at lds_wave_base + 16*l, so a wave moves 1 KB that is contiguous in
// LDS.  lds_wave_base must be the same in every lane.  The copy is tracked by the vector-memory
// counter: wait_vm0() before the data (or a barrier that publishes it) is relied on.
__device__ __forceinline__ void copy16_global_to_lds(const bf16* g_lane, bf16* lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)g_lane,
                                     (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}
__device__ __forceinline__ void wait_vm0() { __builtin_amdgcn_s_waitcnt(0x0F70); }   // vmcnt(0), other counters untouched
// vmcnt(0) and lgkmcnt(0).  The compiler books a copy into LDS against both counters; until it has seen
// both drained it takes the vector-memory queue for out of order and turns every later wait into vmcnt(0).
__device__ __forceinline__ void wait_all_mem() { __builtin_amdgcn_s_waitcnt(0x0070); }

// Rotates a gradient back through the 2-D RoPE: 4 consecutive channels = two (even, odd) pairs, f
// holds their [sin, cos] entries.  Every product and sum is rounded to bf16 like the forward rotation.
__device__ __forceinline__ bf16x4 rope_bwd4(bf16x4 o, bf16x4 f) {
#pragma clang fp contract(off)
    bf16x4 y;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const float s = (float)f[2 * j], c = (float)f[2 * j + 1];
        const float ge = (float)o[2 * j], go = (float)o[2 * j + 1];
        y[2 * j] = (bf16)(rn_bf16(c * ge) + rn_bf16(s * go));
        y[2 * j + 1] = (bf16)(rn_bf16(-s * ge) + rn_bf16(c * go));
    }
    return y;
}

// ints at the end of a (b,h)'s work list (see transpose.hip) that the transpose of many entries uses as
// histogram, then as cursors
__host__ __device__ inline int work_tail_len(int Kb) { return (Kb + 3) & ~3; }
__host__ __device__ inline int fine_chunk(int N) { return N > 16384 ? 256 : 64; }      // llsa_fine_chunk

constexpr int kGroup = 4;      // pooled blocks per LDS buffer in the query-side attention kernels (one per wave)

__device__ __forceinline__ int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// The blocks of the pooled levels a group of query blocks reads, as the forward and the dQ kernel walk them:
// level 1's selected blocks, level 2's, ..., then every block of the coarsest level.  `Level` is llsa_fwd_level
// or llsa_bwd_level (fields sel, T).  Blocks of level l per (b,h): N / 16^(l+1).
struct SharedList {
    int mine;          // lane i: the i-th selected entry over all levels below the coarsest
    int n_listed;      // how many of those there are
    int n_blocks;      // n_listed + blocks of the coarsest level
};
struct SharedBlock {
    int level;         // index into lvl[] (pooled level - 1)
    int64_t tile;      // element offset of the block's tile inside the level's tile array
};
__host__ __device__ inline int64_t coarsest_multiple(int levels) {       // N must be a multiple of 64 * 16^levels
    int64_t m = 64;
    for (int l = 0; l < levels; l++) m *= 16;
    return m;
}
template <typename Level>
__device__ __forceinline__ SharedList shared_list(const Level* lvl, int levels, int N, int bh, int g, int lane) {
    SharedList sl;
    sl.mine = 0;
    int base = 0, nb = N / (kBlk * kBlk);                     // blocks of level 1 per (b,h) = owners of its selection
    int owner = g / kBlk;
    for (int l = 1; l < levels; l++) {
        const int T = lvl[l - 1].T;
        if (lane >= base && lane < base + T) sl.mine = lvl[l - 1].sel[((int64_t)bh * nb + owner) * T + (lane - base)];
        base += T;
        nb /= kBlk;
        owner /= kBlk;
    }
    sl.n_listed = base;
    sl.n_blocks = base + nb;                                  // nb is now the block count of the coarsest level
    return sl;
}
// which entry of lvl[] the i-th block of the walk belongs to (i is wave-uniform)
template <typename Level>
__device__ __forceinline__ int shared_level(const Level* lvl, int levels, int i) {
    int base = 0, l = 1;
    while (l < levels && i >= base + lvl[l - 1].T) {
        base += lvl[l - 1].T;
        l++;
    }
    return l - 1;
}
template <typename Level>
__device__ __forceinline__ SharedBlock shared_block(const SharedList& sl, const Level* lvl, int levels, int N, int bh, int i) {
    SharedBlock sb;
    int base = 0, nb = N / (kBlk * kBlk), l = 1;
    while (l < levels && i >= base + lvl[l - 1].T) {
        base += lvl[l - 1].T;
        nb /= kBlk;
        l++;
    }
    int blk;
    if (l < levels) blk = clampi(__builtin_amdgcn_readlane(sl.mine, i), 0, nb - 1);      // (i < 64 there)
    else blk = i - sl.n_listed;
    sb.level = l - 1;
    sb.tile = ((int64_t)bh * nb + blk) * kTile;
    return sb;
}

// The fine lists of two sibling query blocks (rows ip[0..T) and ip[T..2T), T <= kPairMaxTopk), sorted into
// [blocks both rows name | only the first | only the second]: entry i of that order ends in lane i (2T - n_both
// entries), indices clamped to [0, N1).  n_both is even (an odd common block out is listed once for each row).
// A row that names a block twice shares nothing (n_both = 0).  `scratch`: kWave ints of LDS private to the wave.
constexpr int kPairMaxTopk = 32;
struct PairOrder {
    int mine;
    int n_both;
};
__device__ __forceinline__ PairOrder pair_order(const int* ip, int T, int N1, int lane, int* scratch) {
    const int first = (lane < T) ? clampi(ip[lane], 0, N1 - 1) : -1 - lane;       // (distinct negative fillers)
    const int second = (lane < T) ? clampi(ip[T + lane], 0, N1 - 1) : -65 - lane;
    bool in_second = false, in_first = false, twice = false;
    for (int j = 0; j < T; j++) {
        const int fj = __builtin_amdgcn_readlane(first, j), sj = __builtin_amdgcn_readlane(second, j);
        in_second |= first == sj;
        in_first |= second == fj;
        twice |= (first == fj && lane != j) || (second == sj && lane != j);
    }
    if (__ballot(twice) != 0) in_second = in_first = false;
    unsigned long long both = __ballot(in_second);
    if (__popcll(both) & 1) {
        const int last = 63 - __builtin_clzll(both);
        const int dropped = __builtin_amdgcn_readlane(first, last);
        in_second = in_second && lane != last;
        in_first = in_first && second != dropped;
        both &= ~(1ull << last);
    }
    const int n_both = __popcll(both), n_only = T - n_both;
    const unsigned long long below = (1ull << lane) - 1ull;
    const unsigned long long only1 = __ballot(lane < T && !in_second), only2 = __ballot(lane < T && !in_first);
    if (lane < T) scratch[in_second ? __popcll(both & below) : n_both + __popcll(only1 & below)] = first;
    if (lane < T && !in_first) scratch[n_both + n_only + __popcll(only2 & below)] = second;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    PairOrder po;
    po.mine = scratch[lane];
    po.n_both = n_both;
    return po;
}

// 16- and 8-byte reads that are LDS reads by construction (ds_read_b128 / ds_read_b64)
__device__ __forceinline__ bf16x8 lds_ld16(const bf16* p) {
    return *reinterpret_cast<const __attribute__((address_space(3))) bf16x8*>((const __attribute__((address_space(3))) bf16*)p);
}
__device__ __forceinline__ bf16x4 lds_ld8(const bf16* p) {
    return *reinterpret_cast<const __attribute__((address_space(3))) bf16x4*>((const __attribute__((address_space(3))) bf16*)p);
}
__device__ __forceinline__ void lds_st8(bf16* p, bf16x4 v) {
    *reinterpret_cast<__attribute__((address_space(3))) bf16x4*>((__attribute__((address_space(3))) bf16*)p) = v;
}

// XCD-aware workgroup order.  The 8 XCDs of the chip each have a private L2 and receive
// workgroups round-robin by linear id (id % 8).  Neighbouring logical work items (query or
// key blocks that are close in Z-order) read overlapping K/V/Q rows, so they should share an
// L2: this maps the hardware id to a logical id such that every XCD walks one contiguous
// range of the (x, y) grid.  Returns the logical linear id in [0, gridDim.x * gridDim.y).
constexpr int kXcds = 8;
__device__ __forceinline__ int xcd_logical_id() {
    const int total = gridDim.x * gridDim.y;
    const int lin = blockIdx.y * gridDim.x + blockIdx.x;
    const int xcd = lin % kXcds, slot = lin / kXcds;
    const int q = total / kXcds, rem = total % kXcds;
    return xcd * q + (xcd < rem ? xcd : rem) + slot;
}

}  // namespace llsa
