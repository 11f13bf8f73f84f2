// Index transpose: query-major top-k lists -> key-major CSR (offsets + flat list), used by
// the dK/dV passes.  One workgroup per (b,h) does the whole counting sort in LDS:
// histogram (LDS atomics), exclusive scan, scatter with an LDS cursor, and finally every
// segment is put in ascending query-block order with a per-wave bitmap (set one bit per
// entry, then read the bits back in order), which makes the result -- and therefore the
// accumulation order of dK/dV -- independent of atomic timing.
#include "llsa_device.h"
#include "llsa_host.h"
#include "../../include/llsa_hip.h"

namespace llsa {

constexpr int kTrThreads = 1024;
constexpr int kTrWaves = kTrThreads / kWave;

__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int o = __shfl_up(v, d);
        if (lane >= d) v += o;
    }
    return v;
}

__global__ __launch_bounds__(kTrThreads) void transpose_indices_kernel(const int* __restrict__ idx, int* __restrict__ offsets,
                                                                      int* __restrict__ flat, int Mb, int Kb, int T) {
    HIP_DYNAMIC_SHARED(int, smem)
    const int words = (Mb + 31) / 32;
    int* pos = smem;                               // Kb
    int* wave_tot = smem + Kb;                     // kTrWaves (+ padding to 64)
    unsigned* bitmaps = (unsigned*)(smem + Kb + 64);   // kTrWaves * words

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bh = blockIdx.x;
    const int E = Mb * T;
    idx += (int64_t)bh * E;
    flat += (int64_t)bh * E;
    offsets += (int64_t)bh * (Kb + 1);

    for (int i = tid; i < Kb; i += kTrThreads) pos[i] = 0;
    __syncthreads();
    for (int e = tid; e < E; e += kTrThreads) atomicAdd(&pos[clampi(idx[e], 0, Kb - 1)], 1);
    __syncthreads();

    // exclusive scan over pos[0..Kb): each thread owns `per` consecutive counters
    const int per = (Kb + kTrThreads - 1) / kTrThreads;
    const int c0 = min(tid * per, Kb), c1 = min(c0 + per, Kb);
    int local = 0;
    for (int i = c0; i < c1; i++) local += pos[i];
    const int incl = wave_incl_scan(local, lane);
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    int run = incl - local;
    for (int w = 0; w < wave; w++) run += wave_tot[w];
    for (int i = c0; i < c1; i++) {
        const int c = pos[i];
        offsets[i] = run;
        pos[i] = run;
        run += c;
    }
    if (tid == 0) offsets[Kb] = E;
    __syncthreads();

    for (int e = tid; e < E; e += kTrThreads) {
        const int slot = atomicAdd(&pos[clampi(idx[e], 0, Kb - 1)], 1);
        flat[slot] = e / T;
    }
    __syncthreads();                                // pos[n] is now the END of segment n

    unsigned* bm = bitmaps + wave * words;
    for (int n = wave; n < Kb; n += kTrWaves) {
        const int s = (n == 0) ? 0 : pos[n - 1], e = pos[n];
        if (e - s <= 1) continue;
        for (int w = lane; w < words; w += kWave) bm[w] = 0u;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        for (int i = s + lane; i < e; i += kWave) {
            const int q = flat[i];
            atomicOr(&bm[q >> 5], 1u << (q & 31));
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        int out = s;
        for (int wb = 0; wb < words; wb += kWave) {
            unsigned wd = (wb + lane < words) ? bm[wb + lane] : 0u;
            const int cnt = __popc(wd);
            const int incl2 = wave_incl_scan(cnt, lane);
            int o = out + incl2 - cnt;
            while (wd) {
                const int bit = __ffs((int)wd) - 1;
                flat[o++] = (wb + lane) * 32 + bit;
                wd &= wd - 1;
            }
            out += __shfl(incl2, kWave - 1);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}

}  // namespace llsa

using namespace llsa;

extern "C" int llsa_transpose_indices(const int32_t* idx, int32_t* offsets, int32_t* flat, int B, int H, int Mb, int Kb,
                                      int T, void* stream) {
    LLSA_REQUIRE(idx && offsets && flat, "transpose_indices: null argument");
    LLSA_REQUIRE(B > 0 && H > 0 && Mb > 0 && Kb > 0 && T > 0, "transpose_indices: bad shape");
    const int words = (Mb + 31) / 32;
    const size_t lds = sizeof(int) * ((size_t)Kb + 64 + (size_t)kTrWaves * words);
    LLSA_REQUIRE(lds <= 160 * 1024, "transpose_indices: Kb=%d, Mb=%d need %zu bytes of LDS (limit 163840)", Kb, Mb, lds);
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)transpose_indices_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(-101, "transpose_indices: cannot raise dynamic LDS to %zu bytes: %s", lds, hipGetErrorString(e));
    }
    hipLaunchKernelGGL(transpose_indices_kernel, dim3(B * H), dim3(kTrThreads), lds, (hipStream_t)stream, idx, offsets, flat, Mb, Kb, T);
    return launch_status("transpose_indices");
}
