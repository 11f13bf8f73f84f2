// Bandwidth-bound kernels around the attention: the pooling pyramid (with optional fused
// RoPE and the block-transposed copies the MFMA kernels read), the general mean pool,
// the pooled-gradient accumulation of the backward pass, and the stand-alone RoPE.
#include "llsa_device.h"
#include "llsa_host.h"
#include "../../include/llsa_hip.h"
#include <mutex>

namespace llsa {

// ---------------------------------------------------------------------------------------
// rotation of one 8-channel chunk (4 interleaved pairs) with bf16 rounding after every
// multiply and add, the arithmetic the reference performs in the tensor dtype
// ---------------------------------------------------------------------------------------
//
// Contraction must stay off here: with it the compiler narrows the fp32 expression to bf16
// arithmetic and then fuses multiply and add into one bf16 FMA, i.e. one rounding fewer.
__device__ __forceinline__ bf16x8 rope_chunk_fwd(bf16x8 x, bf16x8 f) {
#pragma clang fp contract(off)
    bf16x8 y;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float s = (float)f[2 * j], c = (float)f[2 * j + 1];
        float xe = (float)x[2 * j], xo = (float)x[2 * j + 1];
        y[2 * j] = (bf16)(rn_bf16(c * xe) - rn_bf16(s * xo));
        y[2 * j + 1] = (bf16)(rn_bf16(s * xe) + rn_bf16(c * xo));
    }
    return y;
}
__device__ __forceinline__ bf16x8 rope_chunk_bwd(bf16x8 g, bf16x8 f) {
#pragma clang fp contract(off)
    bf16x8 y;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float s = (float)f[2 * j], c = (float)f[2 * j + 1];
        float ge = (float)g[2 * j], go = (float)g[2 * j + 1];
        y[2 * j] = (bf16)(rn_bf16(c * ge) + rn_bf16(s * go));
        y[2 * j + 1] = (bf16)(rn_bf16(-s * ge) + rn_bf16(c * go));
    }
    return y;
}

// ---------------------------------------------------------------------------------------
// pooling pyramid: one workgroup = 256 consecutive tokens (16 blocks of 16) of one (b,h) of
// one item.  Thread t owns block r = t/8 and the 8-channel chunk c = t%8: it streams the 16
// rows of its block with 16-byte loads (8 neighbouring lanes cover one 128-byte row), keeps
// them in registers, and emits everything that derives from them: the pooled rows and the
// operand tiles (R and T, see llsa_device.h) the attention kernels read.
// ---------------------------------------------------------------------------------------
struct PoolParams {
    llsa_pool_item it[4];
    const bf16* freq;
    int H, n_items;
};

// The operand tiles of the workgroup's 16 blocks are one contiguous 32 KB piece of the tile
// array.  A thread's registers hold 256-byte pieces of it that are 256 bytes apart from its
// neighbours' (R) or 8-byte pieces scattered over a whole tile (T); stored straight from the
// registers every store instruction would touch 64 different cache lines with 16 or 8 bytes
// each.  They go through LDS instead and leave as full-width stores: thread t of the workgroup
// writes the 16 bytes at (k * 128 + t) * 16 for k = 0..15.  The staging buffer holds the 16-byte
// units of a block in tile order with their low index bits XOR-ed so that both sides spread over
// the banks without padding: exactly 32 KB, five workgroups per CU.
__device__ __forceinline__ int swz_r(int u, int blk) { return u ^ ((u >> 4) ^ (blk & 15)); }   // u = chunk * 16 + row
__device__ __forceinline__ int swz_t(int u) { return u ^ (u >> 5); }                           // u = unit of the T tile

__device__ __forceinline__ void stage_out(bf16* stage, bf16* tiles32k, int t, int n_valid_blocks, bool r_layout) {
    __syncthreads();                              // the staging buffer is filled
#pragma unroll
    for (int k = 0; k < 16; k++) {
        if (k < n_valid_blocks) {
            const int u = r_layout ? swz_r(t, k) : swz_t(t);
            st16(tiles32k + (k * 128 + t) * 8, ld16(stage + (k * 128 + u) * 8));
        }
    }
    __syncthreads();                              // and may be refilled
}

// RMS normalisation of the thread's 16 rows (8 channels of each; the row's other channels are
// in the 7 neighbouring lanes): x <- bf16(x * rsqrt(mean(x^2) + eps) * gamma), in fp32.
__device__ __forceinline__ void rms_norm_rows(bf16x8 xv[16], const float* gamma, float eps, int c) {
    float g[8];
#pragma unroll
    for (int e = 0; e < 8; e++) g[e] = gamma[c * 8 + e];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) ss += (float)xv[i][e] * (float)xv[i][e];
        ss += __shfl_xor(ss, 1);
        ss += __shfl_xor(ss, 2);
        ss += __shfl_xor(ss, 4);
        const float rstd = rsqrtf(ss * (1.f / kD) + eps);
#pragma unroll
        for (int e = 0; e < 8; e++) xv[i][e] = (bf16)((float)xv[i][e] * rstd * g[e]);
    }
}

template <bool NORM>
__global__ __launch_bounds__(128) void pool_pyramid_kernel(PoolParams p) {
    __shared__ __align__(16) bf16 stage[16 * 128 * 8];
    // (items interleaved along x: q and k with their rotation are arithmetic-heavy, v with its two tiles is store-heavy,
    // and workgroups start in x order -- a launch that runs one item after the other works in phases)
    const int item = (int)blockIdx.x % p.n_items, bx = (int)blockIdx.x / p.n_items;
    const llsa_pool_item& it = p.it[item];
    const int n1 = it.n / kBlk;
    if (bx * 16 >= n1) return;                    // uniform over the workgroup
    const int bh = blockIdx.y, b = bh / p.H, h = bh % p.H;
    const int t = threadIdx.x, c = t & 7, r = t >> 3;
    const int blk = bx * 16 + r;
    const bool valid = blk < n1;
    const int n_valid = min(16, n1 - bx * 16);

    bf16x8 xv[16];
    bf16x8 y = zero8();
    if (valid) {
        const bf16* x = (const bf16*)it.x + b * it.sxb + h * it.sxh + (int64_t)blk * kBlk * it.sxn + c * 8;
#pragma unroll
        for (int i = 0; i < 16; i++) xv[i] = ld16(x + i * it.sxn);
        if (NORM && it.gamma != nullptr) rms_norm_rows(xv, it.gamma, it.eps, c);
        if (it.rope) {
            const bf16* f = p.freq + ((int64_t)blk * kBlk) * kD + c * 8;
#pragma unroll
            for (int i = 0; i < 16; i++) xv[i] = rope_chunk_fwd(xv[i], ld16(f + i * kD));
        }
        if (it.xrot != nullptr) {        // the rows as the attention sees them (normalised, rotated), row-major
            bf16* xo = (bf16*)it.xrot + ((int64_t)bh * it.n + (int64_t)blk * kBlk) * kD + c * 8;
#pragma unroll
            for (int i = 0; i < 16; i++) st16(xo + i * kD, xv[i]);
        }
        if (it.y1 != nullptr || it.y2 != nullptr || it.y1r != nullptr || it.y1t != nullptr) {
            float acc[8];
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] = 0.f;
#pragma unroll
            for (int i = 0; i < 16; i++)
#pragma unroll
                for (int e = 0; e < 8; e++) acc[e] = rn_bf16(acc[e] + (float)xv[i][e]);
#pragma unroll
            for (int e = 0; e < 8; e++) y[e] = (bf16)(acc[e] * 0.0625f);
            if (it.y1 != nullptr) st16((bf16*)it.y1 + ((int64_t)bh * n1 + blk) * kD + c * 8, y);
        }
    }
    if (it.xr != nullptr) {              // R tile: chunk c of row i is 16-byte unit c * 16 + i of the block
        if (valid) {
#pragma unroll
            for (int i = 0; i < 16; i++) st16(stage + (r * 128 + swz_r(c * 16 + i, r)) * 8, xv[i]);
        }
        stage_out(stage, (bf16*)it.xr + ((int64_t)bh * n1 + bx * 16) * kTile, t, n_valid, true);
    }
    if (it.xt != nullptr) {              // T tile: channels 8c+e, 8c+e+1 of tokens 4q..4q+3 are one 16-byte unit
        if (valid) {
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int ep = 0; ep < 4; ep++) {
                    bf16x8 v;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        v[j] = xv[4 * q + j][2 * ep];
                        v[4 + j] = xv[4 * q + j][2 * ep + 1];
                    }
                    const int u = t_tile_off(4 * q, 8 * c + 2 * ep) / 8;      // 16-byte unit inside the tile
                    st16(stage + (r * 128 + swz_t(u)) * 8, v);
                }
        }
        stage_out(stage, (bf16*)it.xt + ((int64_t)bh * n1 + bx * 16) * kTile, t, n_valid, false);
    }
    if (it.y2 == nullptr && it.y1r == nullptr && it.y1t == nullptr && it.y2r == nullptr && it.y2t == nullptr) return;   // uniform over the workgroup

    // the 16 pooled rows of this workgroup are one block of the next level
    bf16 (*sm)[kD] = reinterpret_cast<bf16 (*)[kD]>(stage);
    st16(&sm[r][c * 8], y);
    __syncthreads();
    const int n2 = it.n / (kBlk * kBlk);
    if ((it.y2 != nullptr || it.y2r != nullptr || it.y2t != nullptr) && t < 8) {
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] = 0.f;
        for (int i = 0; i < 16; i++) {
            bf16x8 v = ld16(&sm[i][t * 8]);
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] = rn_bf16(acc[e] + (float)v[e]);
        }
        bf16x8 y2;
#pragma unroll
        for (int e = 0; e < 8; e++) y2[e] = (bf16)(acc[e] * 0.0625f);
        if (it.y2 != nullptr) st16((bf16*)it.y2 + ((int64_t)bh * n2 + bx) * kD + t * 8, y2);
        // this workgroup's level-2 row is row bx % 16 of level-2 block bx / 16: its 8-channel chunk
        // t goes straight into that block's tiles (the other 15 rows come from the neighbouring workgroups)
        const int64_t tile2 = ((int64_t)bh * (n2 / kBlk) + bx / kBlk) * kTile;
        const int r2 = bx % kBlk;
        if (it.y2r != nullptr) st16((bf16*)it.y2r + tile2 + (t * 16 + r2) * 8, y2);
        if (it.y2t != nullptr) {
#pragma unroll
            for (int e = 0; e < 8; e++) ((bf16*)it.y2t)[tile2 + t_tile_off(r2, t * 8 + e)] = y2[e];
        }
    }
    if (it.y1r != nullptr)               // thread (r, c) holds chunk c of pooled row r
        st16((bf16*)it.y1r + ((int64_t)bh * n2 + bx) * kTile + (c * 16 + r) * 8, y);
    if (it.y1t != nullptr) {             // thread -> (channel ch, token half)
        const int ch = t & 63, half = t >> 6;
#pragma unroll
        for (int q = 0; q < 2; q++) {
            bf16x4 v;
#pragma unroll
            for (int j = 0; j < 4; j++) v[j] = sm[half * 8 + q * 4 + j][ch];
            st8((bf16*)it.y1t + ((int64_t)bh * n2 + bx) * kTile + t_tile_off(half * 8 + q * 4, ch), v);
        }
    }
}

// ---------------------------------------------------------------------------------------
// general mean pool (any K, C, strides), one thread per output element
// ---------------------------------------------------------------------------------------
struct Strides4 {
    int64_t s[4];
};

template <typename T>
__global__ void mean_pool_fwd_kernel(const T* x, Strides4 sx, T* y, Strides4 sy, int H, int C, int K) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int s = blockIdx.y, bh = blockIdx.z, b = bh / H, h = bh % H;
    const T* xp = x + b * sx.s[0] + h * sx.s[1] + (int64_t)s * K * sx.s[2] + c * sx.s[3];
    float acc = 0.f;
    for (int i = 0; i < K; i++) acc = (float)(T)(acc + (float)xp[i * sx.s[2]]);
    y[b * sy.s[0] + h * sy.s[1] + s * sy.s[2] + c * sy.s[3]] = (T)(acc / (float)K);
}

template <typename T>
__global__ void mean_pool_bwd_kernel(const T* dy, Strides4 sdy, T* dx, Strides4 sdx, int H, int C, int K) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int s = blockIdx.y, bh = blockIdx.z, b = bh / H, h = bh % H;
    const T g = (T)((float)dy[b * sdy.s[0] + h * sdy.s[1] + s * sdy.s[2] + c * sdy.s[3]] / (float)K);
    T* xp = dx + b * sdx.s[0] + h * sdx.s[1] + (int64_t)s * K * sdx.s[2] + c * sdx.s[3];
    for (int i = 0; i < K; i++) xp[i * sdx.s[2]] = g;
}

// ---------------------------------------------------------------------------------------
// pooled-gradient accumulation: out = rn(dx + rn(g1/16)), g1 = dy1 or rn(dy1 + rn(dy2/16)),
// optionally rotated back.  One thread per (token, 8-channel chunk).
// ---------------------------------------------------------------------------------------
struct Strides3 {
    int64_t b, h, n;
};

__global__ __launch_bounds__(256) void pool_bwd_accum_kernel(const bf16* dx, Strides3 sdx, const bf16* dy1,
                                                             const bf16* dy2, bf16* out, Strides3 so,
                                                             const bf16* freq, int H, int N) {
    const int tok = blockIdx.x * 32 + (threadIdx.x >> 3), c = threadIdx.x & 7;
    if (tok >= N) return;
    const int bh = blockIdx.y, b = bh / H, h = bh % H;
    const int n1 = N / kBlk, n2 = n1 / kBlk;
    bf16x8 g1 = ld16(dy1 + ((int64_t)bh * n1 + tok / kBlk) * kD + c * 8);
    if (dy2 != nullptr) {
        bf16x8 g2 = ld16(dy2 + ((int64_t)bh * n2 + tok / (kBlk * kBlk)) * kD + c * 8);
#pragma unroll
        for (int e = 0; e < 8; e++) g1[e] = (bf16)((float)g1[e] + rn_bf16((float)g2[e] * 0.0625f));
    }
    bf16x8 x = ld16(dx + b * sdx.b + h * sdx.h + (int64_t)tok * sdx.n + c * 8);
#pragma unroll
    for (int e = 0; e < 8; e++) x[e] = (bf16)((float)x[e] + rn_bf16((float)g1[e] * 0.0625f));
    if (freq != nullptr) x = rope_chunk_bwd(x, ld16(freq + (int64_t)tok * kD + c * 8));
    st16(out + b * so.b + h * so.h + (int64_t)tok * so.n + c * 8, x);
}

// ---------------------------------------------------------------------------------------
// stand-alone RoPE: one thread per (token, 8-channel chunk), 32 tokens per workgroup
// ---------------------------------------------------------------------------------------
template <bool BWD>
__global__ __launch_bounds__(256) void rope_kernel(const bf16* x, Strides3 sx, const bf16* freq, bf16* y,
                                                   Strides3 sy, int H, int S) {
    const int tok = blockIdx.x * 32 + (threadIdx.x >> 3), c = threadIdx.x & 7;
    if (tok >= S) return;
    const int bh = blockIdx.y, b = bh / H, h = bh % H;
    bf16x8 v = ld16(x + b * sx.b + h * sx.h + (int64_t)tok * sx.n + c * 8);
    bf16x8 f = ld16(freq + (int64_t)tok * kD + c * 8);
    v = BWD ? rope_chunk_bwd(v, f) : rope_chunk_fwd(v, f);
    st16(y + b * sy.b + h * sy.h + (int64_t)tok * sy.n + c * 8, v);
}

// ---------------------------------------------------------------------------------------
// Backward of the RMS normalisation.  Thread mapping of the stand-alone RoPE: one thread per
// (token, 8-channel chunk), 32 tokens at a time, kNormTokens tokens per workgroup; a workgroup
// also sums dy * xn over its tokens (fixed order) into one row of `partials`, which
// rmsnorm_dgamma_kernel adds up.
// ---------------------------------------------------------------------------------------
constexpr int kNormTokens = 256;
constexpr int kGammaGroups = 64;

__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(const bf16* dy, Strides3 sdy, const bf16* x, Strides3 sx,
                                                          const float* __restrict__ gamma, float eps, bf16* dx, Strides3 sdx,
                                                          float* __restrict__ partials, int H, int N) {
    __shared__ float red[32][kD];
    const int row = threadIdx.x >> 3, c = threadIdx.x & 7;
    const int bh = blockIdx.y, b = bh / H, h = bh % H;
    float contrib[8], gam[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
        contrib[e] = 0.f;
        gam[e] = gamma[c * 8 + e];
    }
#pragma unroll 2
    for (int it = 0; it < kNormTokens / 32; it++) {
        const int tok = blockIdx.x * kNormTokens + it * 32 + row;
        if (tok >= N) break;
        const bf16x8 xv = ld16(x + b * sx.b + h * sx.h + (int64_t)tok * sx.n + c * 8);
        const bf16x8 gv = ld16(dy + b * sdy.b + h * sdy.h + (int64_t)tok * sdy.n + c * 8);
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) ss += (float)xv[e] * (float)xv[e];
        ss += __shfl_xor(ss, 1);
        ss += __shfl_xor(ss, 2);
        ss += __shfl_xor(ss, 4);
        const float rstd = rsqrtf(ss * (1.f / kD) + eps);
        float xn[8], g[8], dot = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            xn[e] = (float)xv[e] * rstd;
            g[e] = (float)gv[e] * gam[e];
            dot += g[e] * xn[e];
            contrib[e] += (float)gv[e] * xn[e];
        }
        dot += __shfl_xor(dot, 1);
        dot += __shfl_xor(dot, 2);
        dot += __shfl_xor(dot, 4);
        dot *= 1.f / kD;
        bf16x8 o;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] = (bf16)(rstd * (g[e] - xn[e] * dot));
        st16(dx + b * sdx.b + h * sdx.h + (int64_t)tok * sdx.n + c * 8, o);
    }
#pragma unroll
    for (int e = 0; e < 8; e++) red[row][c * 8 + e] = contrib[e];
    __syncthreads();
    if (threadIdx.x < kD) {
        float s = 0.f;
        for (int r = 0; r < 32; r++) s += red[r][threadIdx.x];
        partials[((int64_t)bh * gridDim.x + blockIdx.x) * kD + threadIdx.x] = s;
    }
}

// Workgroup g of G adds rows g, g + G, g + 2G, ... of `partials` (thread (j, ch) every fourth of
// them, then the four j's) into row g of `out`.  With out == partials a workgroup overwrites a
// row that only it has read, so a first launch with G workgroups can fold the rows in place and
// a second with one workgroup finishes.
__global__ __launch_bounds__(256) void rmsnorm_dgamma_kernel(const float* partials, float* out, int64_t rows) {
    __shared__ float red[4][kD];
    const int ch = threadIdx.x & 63, j = threadIdx.x >> 6;
    const int64_t G = gridDim.x;
    float s = 0.f;
    for (int64_t r = blockIdx.x + j * G; r < rows; r += 4 * G) s += partials[r * kD + ch];
    red[j][ch] = s;
    __syncthreads();
    if (j == 0) out[blockIdx.x * kD + ch] = (red[0][ch] + red[1][ch]) + (red[2][ch] + red[3][ch]);
}

}  // namespace llsa

using namespace llsa;

extern "C" int llsa_pool_pyramid_fwd(const llsa_pool_item* items, int n_items, const void* freq, int B, int H,
                                     void* stream) {
    LLSA_REQUIRE(items != nullptr && n_items >= 1 && n_items <= 4, "pool_pyramid: 1..4 items, got %d", n_items);
    LLSA_REQUIRE(B > 0 && H > 0, "pool_pyramid: bad B/H");
    PoolParams p;
    p.freq = (const bf16*)freq;
    p.H = H;
    int max_n = 0;
    for (int i = 0; i < n_items; i++) {
        const llsa_pool_item& it = items[i];
        LLSA_REQUIRE(it.x != nullptr && it.n > 0 && it.n % 16 == 0, "pool_pyramid: item %d: n=%d must be a positive multiple of 16", i, it.n);
        LLSA_REQUIRE(aligned16(it.x) && stride_ok(it.sxb) && stride_ok(it.sxh) && stride_ok(it.sxn),
                     "pool_pyramid: item %d: rows must be 16-byte aligned", i);
        LLSA_REQUIRE((it.y2 == nullptr && it.y1t == nullptr && it.y1r == nullptr) || it.n % 256 == 0,
                     "pool_pyramid: item %d: level-2 outputs need n %% 256 == 0 (n=%d)", i, it.n);
        LLSA_REQUIRE((it.y2r == nullptr && it.y2t == nullptr) || it.n % 4096 == 0,
                     "pool_pyramid: item %d: level-2 tiles need n %% 4096 == 0 (n=%d)", i, it.n);
        LLSA_REQUIRE(aligned16(it.y2r) && aligned16(it.y2t), "pool_pyramid: item %d: outputs must be 16-byte aligned", i);
        LLSA_REQUIRE(!it.rope || freq != nullptr, "pool_pyramid: item %d: rope needs freq", i);
        LLSA_REQUIRE(it.gamma == nullptr || it.eps >= 0.f, "pool_pyramid: item %d: eps must be >= 0", i);
        LLSA_REQUIRE(aligned16(it.y1) && aligned16(it.y2) && aligned16(it.xr) && aligned16(it.xt) && aligned16(it.y1r) &&
                         aligned16(it.y1t) && aligned16(it.xrot),
                     "pool_pyramid: item %d: outputs must be 16-byte aligned", i);
        p.it[i] = it;
        if (it.n > max_n) max_n = it.n;
    }
    for (int i = n_items; i < 4; i++) p.it[i] = items[0];
    bool norm = false;
    for (int i = 0; i < n_items; i++) norm = norm || items[i].gamma != nullptr;
    p.n_items = n_items;
    dim3 grid((max_n + 255) / 256 * n_items, B * H);
    if (norm)
        hipLaunchKernelGGL(HIP_KERNEL_NAME(pool_pyramid_kernel<true>), grid, dim3(128), 0, (hipStream_t)stream, p);
    else
        hipLaunchKernelGGL(HIP_KERNEL_NAME(pool_pyramid_kernel<false>), grid, dim3(128), 0, (hipStream_t)stream, p);
    return launch_status("pool_pyramid");
}

template <typename T>
static int mean_pool_launch(bool bwd, const void* a, const int64_t* sa, void* o, const int64_t* so, int B, int H,
                            int S_out, int C, int K, hipStream_t st) {
    Strides4 s1, s2;
    for (int i = 0; i < 4; i++) {
        s1.s[i] = sa[i];
        s2.s[i] = so[i];
    }
    dim3 grid((C + 63) / 64, S_out, B * H);
    if (!bwd)
        hipLaunchKernelGGL(HIP_KERNEL_NAME(mean_pool_fwd_kernel<T>), grid, dim3(64), 0, st, (const T*)a, s1, (T*)o, s2, H, C, K);
    else
        hipLaunchKernelGGL(HIP_KERNEL_NAME(mean_pool_bwd_kernel<T>), grid, dim3(64), 0, st, (const T*)a, s1, (T*)o, s2, H, C, K);
    return launch_status("mean_pool");
}

extern "C" int llsa_mean_pool_fwd(const void* x, const int64_t* sx, void* y, const int64_t* sy, int B, int H, int S,
                                  int C, int K, int dtype, void* stream) {
    LLSA_REQUIRE(x && y && sx && sy, "mean_pool_fwd: null argument");
    LLSA_REQUIRE(B > 0 && H > 0 && C > 0 && K > 0 && S > 0 && S % K == 0, "mean_pool_fwd: S=%d must be a positive multiple of K=%d", S, K);
    LLSA_REQUIRE(S / K <= 65535 && B * H <= 65535, "mean_pool_fwd: grid too large");
    if (dtype == LLSA_DTYPE_BF16) return mean_pool_launch<bf16>(false, x, sx, y, sy, B, H, S / K, C, K, (hipStream_t)stream);
    if (dtype == LLSA_DTYPE_F32) return mean_pool_launch<float>(false, x, sx, y, sy, B, H, S / K, C, K, (hipStream_t)stream);
    return fail(-2, "mean_pool_fwd: unsupported dtype %d", dtype);
}

extern "C" int llsa_mean_pool_bwd(const void* dy, const int64_t* sdy, void* dx, const int64_t* sdx, int B, int H,
                                  int S_out, int C, int K, int dtype, void* stream) {
    LLSA_REQUIRE(dy && dx && sdy && sdx, "mean_pool_bwd: null argument");
    LLSA_REQUIRE(B > 0 && H > 0 && C > 0 && K > 0 && S_out > 0, "mean_pool_bwd: bad shape");
    LLSA_REQUIRE(S_out <= 65535 && B * H <= 65535, "mean_pool_bwd: grid too large");
    if (dtype == LLSA_DTYPE_BF16) return mean_pool_launch<bf16>(true, dy, sdy, dx, sdx, B, H, S_out, C, K, (hipStream_t)stream);
    if (dtype == LLSA_DTYPE_F32) return mean_pool_launch<float>(true, dy, sdy, dx, sdx, B, H, S_out, C, K, (hipStream_t)stream);
    return fail(-2, "mean_pool_bwd: unsupported dtype %d", dtype);
}

static bool s3_ok(const int64_t* s) { return stride_ok(s[0]) && stride_ok(s[1]) && stride_ok(s[2]); }

extern "C" int llsa_pool_bwd_accum(const void* dx, const int64_t* sdx, const void* dy1, const void* dy2, void* out,
                                   const int64_t* sout, const void* freq, int B, int H, int N, void* stream) {
    LLSA_REQUIRE(dx && dy1 && out && sdx && sout, "pool_bwd_accum: null argument");
    LLSA_REQUIRE(N > 0 && N % 16 == 0 && (dy2 == nullptr || N % 256 == 0), "pool_bwd_accum: bad N=%d", N);
    LLSA_REQUIRE(aligned16(dx) && aligned16(dy1) && aligned16(dy2) && aligned16(out) && aligned16(freq) && s3_ok(sdx) && s3_ok(sout),
                 "pool_bwd_accum: rows must be 16-byte aligned");
    Strides3 a{sdx[0], sdx[1], sdx[2]}, o{sout[0], sout[1], sout[2]};
    hipLaunchKernelGGL(pool_bwd_accum_kernel, dim3((N + 31) / 32, B * H), dim3(256), 0, (hipStream_t)stream, (const bf16*)dx, a,
                       (const bf16*)dy1, (const bf16*)dy2, (bf16*)out, o, (const bf16*)freq, H, N);
    return launch_status("pool_bwd_accum");
}

static int rope_launch(bool bwd, const void* x, const int64_t* sx, const void* freq, void* y, const int64_t* sy, int B,
                       int H, int S, void* stream) {
    LLSA_REQUIRE(x && y && freq && sx && sy, "rope: null argument");
    LLSA_REQUIRE(B > 0 && H > 0 && S > 0, "rope: bad shape");
    LLSA_REQUIRE(aligned16(x) && aligned16(y) && aligned16(freq) && s3_ok(sx) && s3_ok(sy), "rope: rows must be 16-byte aligned");
    Strides3 a{sx[0], sx[1], sx[2]}, o{sy[0], sy[1], sy[2]};
    dim3 grid((S + 31) / 32, B * H);
    if (bwd)
        hipLaunchKernelGGL(HIP_KERNEL_NAME(rope_kernel<true>), grid, dim3(256), 0, (hipStream_t)stream, (const bf16*)x, a,
                           (const bf16*)freq, (bf16*)y, o, H, S);
    else
        hipLaunchKernelGGL(HIP_KERNEL_NAME(rope_kernel<false>), grid, dim3(256), 0, (hipStream_t)stream, (const bf16*)x, a,
                           (const bf16*)freq, (bf16*)y, o, H, S);
    return launch_status("rope");
}

extern "C" int llsa_rope_fwd(const void* x, const int64_t* sx, const void* freq, void* y, const int64_t* sy, int B, int H,
                             int S, void* stream) {
    return rope_launch(false, x, sx, freq, y, sy, B, H, S, stream);
}
extern "C" int llsa_rope_bwd(const void* dy, const int64_t* sdy, const void* freq, void* dx, const int64_t* sdx, int B,
                             int H, int S, void* stream) {
    return rope_launch(true, dy, sdy, freq, dx, sdx, B, H, S, stream);
}

// ---------------------------------------------------------------------------------------
// Token permutation: y[b, i, :] = x[b, index[i], :] for rows of `chunks` 16-byte pieces.  A
// workgroup takes 256 consecutive pieces of the output, so stores are contiguous and every
// source row is read in pieces of at least min(row, 4 KB).  An index outside [0, n_in) gives a
// row of zeros.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void gather_rows_kernel(const i32x4* __restrict__ x, i32x4* __restrict__ y,
                                                          const int32_t* __restrict__ index, int n_out, int n_in, int chunks,
                                                          int64_t x_batch, int64_t y_batch) {
    const int64_t piece = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (piece >= (int64_t)n_out * chunks) return;
    const int row = (int)(piece / chunks), c = (int)(piece - (int64_t)row * chunks);
    const int src = index[row];
    i32x4 v = {0, 0, 0, 0};
    if ((unsigned)src < (unsigned)n_in) v = x[blockIdx.y * x_batch + (int64_t)src * chunks + c];
    y[blockIdx.y * y_batch + piece] = v;
}

extern "C" int llsa_gather_rows(const void* x, void* y, const int32_t* index, int B, int n_out, int n_in, int row_bytes,
                                int64_t x_batch_bytes, int64_t y_batch_bytes, void* stream) {
    LLSA_REQUIRE(x && y && index, "gather_rows: null argument");
    LLSA_REQUIRE(B > 0 && n_out > 0 && n_in > 0 && row_bytes > 0 && row_bytes % 16 == 0, "gather_rows: rows must be a multiple of 16 bytes");
    LLSA_REQUIRE(aligned16(x) && aligned16(y) && x_batch_bytes % 16 == 0 && y_batch_bytes % 16 == 0 &&
                     x_batch_bytes >= (int64_t)n_in * row_bytes && y_batch_bytes >= (int64_t)n_out * row_bytes,
                 "gather_rows: batches must be 16-byte aligned and hold their rows");
    LLSA_REQUIRE(B <= 65535, "gather_rows: at most 65535 batches");
    const int chunks = row_bytes / 16;
    const int64_t pieces = (int64_t)n_out * chunks;
    LLSA_REQUIRE(pieces < ((int64_t)1 << 31) * 256, "gather_rows: too many rows");
    hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)((pieces + 255) / 256), B), dim3(256), 0, (hipStream_t)stream,
                       (const i32x4*)x, (i32x4*)y, index, n_out, n_in, chunks, x_batch_bytes / 16, y_batch_bytes / 16);
    return launch_status("gather_rows");
}

extern "C" int64_t llsa_rmsnorm_bwd_partials(int B, int H, int N) {
    if (B <= 0 || H <= 0 || N <= 0) return -1;
    return (int64_t)B * H * ((N + kNormTokens - 1) / kNormTokens) * kD;
}

static int rmsnorm_bwd_launch(const void* dy, const int64_t* sdy, const void* x, const int64_t* sx, const float* gamma, float eps,
                              void* dx, const int64_t* sdx, float* dgamma, float* partials, int B, int H, int N, void* stream) {
    LLSA_REQUIRE(dy && x && gamma && dx && dgamma && partials && sdy && sx && sdx, "rmsnorm_bwd: null argument");
    LLSA_REQUIRE(B > 0 && H > 0 && N > 0 && eps >= 0.f, "rmsnorm_bwd: bad shape or eps");
    LLSA_REQUIRE(aligned16(dy) && aligned16(x) && aligned16(dx) && s3_ok(sdy) && s3_ok(sx) && s3_ok(sdx),
                 "rmsnorm_bwd: rows must be 16-byte aligned");
    Strides3 a{sdy[0], sdy[1], sdy[2]}, bx{sx[0], sx[1], sx[2]}, o{sdx[0], sdx[1], sdx[2]};
    const int parts = (N + kNormTokens - 1) / kNormTokens;
    int64_t rows = (int64_t)B * H * parts;
    hipLaunchKernelGGL(rmsnorm_bwd_kernel, dim3(parts, B * H), dim3(256), 0, (hipStream_t)stream, (const bf16*)dy, a, (const bf16*)x, bx,
                       gamma, eps, (bf16*)dx, o, partials, H, N);
    if (rows > 4 * kGammaGroups) {
        hipLaunchKernelGGL(rmsnorm_dgamma_kernel, dim3(kGammaGroups), dim3(256), 0, (hipStream_t)stream, (const float*)partials,
                           partials, rows);
        rows = kGammaGroups;
    }
    hipLaunchKernelGGL(rmsnorm_dgamma_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, (const float*)partials, dgamma, rows);
    return launch_status("rmsnorm_bwd");
}

extern "C" int llsa_rmsnorm_bwd(const void* dy, const int64_t* sdy, const void* x, const int64_t* sx, const float* gamma, float eps,
                                void* dx, const int64_t* sdx, float* dgamma, float* partials, int B, int H, int N, void* stream) {
    return rmsnorm_bwd_launch(dy, sdy, x, sx, gamma, eps, dx, sdx, dgamma, partials, B, H, N, stream);
}

// ---------------------------------------------------------------------------------------
// The same backward for callers that cannot allocate (a step under HIP graph capture, a tight
// serving loop): the per-workgroup partial sums of dgamma live in a static device array instead
// of a buffer the caller brings.  Every GPU holds its own copy of the array at its own address;
// the address is looked up once per device, with that device current, and the kernels receive
// it as an ordinary pointer argument.
// ---------------------------------------------------------------------------------------
static __device__ __align__(256) float scratch[LLSA_STATIC_PARTIALS_MAX];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices];       // device address of `scratch` per device ordinal, looked up on first use
}  // namespace

extern "C" int llsa_rmsnorm_bwd_static(const void* dy, const int64_t* sdy, const void* x, const int64_t* sx, const float* gamma,
                                       float eps, void* dx, const int64_t* sdx, float* dgamma, int B, int H, int N, void* stream) {
    const int64_t need = llsa_rmsnorm_bwd_partials(B, H, N);
    LLSA_REQUIRE(need > 0, "rmsnorm_bwd_static: bad shape");
    LLSA_REQUIRE(need <= (int64_t)LLSA_STATIC_PARTIALS_MAX,
                 "rmsnorm_bwd_static: B*H*ceil(N/256)*64 = %lld partial sums exceed the static scratch of %lld floats; "
                 "use llsa_rmsnorm_bwd with a caller-owned buffer",
                 (long long)need, (long long)LLSA_STATIC_PARTIALS_MAX);
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(-102, "rmsnorm_bwd_static: hipGetDevice: %s", hipGetErrorString(e));
    LLSA_REQUIRE(dev >= 0 && dev < kMaxDevices, "rmsnorm_bwd_static: device ordinal %d out of range", dev);
    float* part = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (g_scratch_ptr[dev] == nullptr) {
            void* p = nullptr;
            e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess || p == nullptr)
                return fail(-103, "rmsnorm_bwd_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
            g_scratch_ptr[dev] = (float*)p;
        }
        part = g_scratch_ptr[dev];
    }
    // every row of the partial sums this call reads is written by its first kernel, so nothing has to be cleared
    return rmsnorm_bwd_launch(dy, sdy, x, sx, gamma, eps, dx, sdx, dgamma, part, B, H, N, stream);
}
