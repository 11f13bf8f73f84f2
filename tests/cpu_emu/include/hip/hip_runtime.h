// CPU stand-in for <hip/hip_runtime.h>, used ONLY by the test build under tests/cpu_emu.
//
// The HIP sources of llsa_amd/csrc are compiled unchanged for x86 with this header on the
// include path instead of ROCm's.  Every thread of a workgroup becomes a ucontext fiber;
// wave-collective operations (shuffles, MFMA) and barriers are rendezvous points between
// fibers.  This gives a host build of the kernels that runs under gdb / AddressSanitizer at
// tiny sizes, so index arithmetic and operand layouts can be checked without a GPU.
// It is test infrastructure: the product library (libllsa_hip.so) never contains it.
#pragma once
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __shared__ static
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
#define HIP_KERNEL_NAME(...) __VA_ARGS__
#define HIP_DYNAMIC_SHARED(type, var) type* var = reinterpret_cast<type*>(emu::dyn_smem());

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
struct uint3_emu { unsigned x, y, z; };

typedef void* hipStream_t;
typedef int hipError_t;
#define hipSuccess 0
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipPeekAtLastError() { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "emu"; }
inline hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
#define HIP_SYMBOL(x) x
template <typename T>
inline hipError_t hipGetSymbolAddress(void** p, T& symbol) { *p = (void*)&symbol; return hipSuccess; }
inline hipError_t hipMemsetAsync(void* p, int v, size_t n, hipStream_t) { memset(p, v, n); return hipSuccess; }

namespace emu {
extern uint3_emu g_threadIdx, g_blockIdx;
extern dim3 g_blockDim, g_gridDim;
void launch(dim3 grid, dim3 block, size_t shmem, const std::function<void()>& body);
void* dyn_smem();
void block_barrier();
void wave_sync();   // lock-step point: on the GPU a wave executes in lock step, fibers do not
uint32_t shfl_u32(uint32_t v, int src_lane);
uint64_t ballot(bool pred);
int lane_id();
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
f32x4_t mfma_16x16x32_bf16(bf16x8_t a, bf16x8_t b, f32x4_t c);
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
s16x4_t ds_read_tr16_b64(const void* p);
}  // namespace emu

#define threadIdx emu::g_threadIdx
#define blockIdx emu::g_blockIdx
#define blockDim emu::g_blockDim
#define gridDim emu::g_gridDim

#define hipLaunchKernelGGL(kern, grid, block, shmem, stream, ...) \
    emu::launch(dim3(grid), dim3(block), (shmem), [&]() { kern(__VA_ARGS__); })

inline void __syncthreads() { emu::block_barrier(); }

template <typename T>
inline T __shfl(T v, int src, int width = 64) {
    static_assert(sizeof(T) == 4, "emu shuffles are 32-bit");
    uint32_t u;
    memcpy(&u, &v, 4);
    int lane = emu::lane_id();
    int base = lane & ~(width - 1);
    u = emu::shfl_u32(u, base + (src & (width - 1)));
    T r;
    memcpy(&r, &u, 4);
    return r;
}
template <typename T>
inline T __shfl_xor(T v, int mask, int width = 64) {
    return __shfl(v, (emu::lane_id() ^ mask) & (width - 1), width);
}
template <typename T>
inline T __shfl_down(T v, unsigned d, int width = 64) {
    int l = emu::lane_id() & (width - 1);
    return __shfl(v, (l + (int)d < width) ? l + (int)d : l, width);
}
template <typename T>
inline T __shfl_up(T v, unsigned d, int width = 64) {
    int l = emu::lane_id() & (width - 1);
    return __shfl(v, (l >= (int)d) ? l - (int)d : l, width);
}
inline uint64_t __ballot(int pred) { return emu::ballot(pred != 0); }
// v_permlane16_swap / v_permlane32_swap of gfx950: rows of 16 lanes [r0 r1 r2 r3] of a and [s0 s1 s2 s3] of b become
// a' = [r0 s0 r2 s2], b' = [r1 s1 r3 s3]; halves of 32 lanes [a_lo a_hi], [b_lo b_hi] become a' = [a_lo b_lo], b' = [a_hi b_hi]
typedef __attribute__((ext_vector_type(2))) unsigned emu_u32x2;
inline emu_u32x2 emu_permlane_swap(unsigned a, unsigned b, int width) {
    const int l = emu::lane_id();
    const bool upper = (l & width) != 0;
    const unsigned b_below = __shfl(b, (l - width) & 63), a_above = __shfl(a, (l + width) & 63);
    emu_u32x2 r;
    r[0] = upper ? b_below : a;
    r[1] = upper ? b : a_above;
    return r;
}
#define __builtin_amdgcn_permlane16_swap(a, b, fi, bc) emu_permlane_swap((a), (b), 16)
#define __builtin_amdgcn_permlane32_swap(a, b, fi, bc) emu_permlane_swap((a), (b), 32)
inline int __popcll(unsigned long long x) { return __builtin_popcountll(x); }
inline int __popc(unsigned x) { return __builtin_popcount(x); }
inline int __ffsll(unsigned long long x) { return __builtin_ffsll(x); }
inline int __ffs(int x) { return __builtin_ffs(x); }
inline int __clz(int x) { return x ? __builtin_clz((unsigned)x) : 32; }

#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) emu::mfma_16x16x32_bf16((a), (b), (c))
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) emu::ds_read_tr16_b64((const void*)(p))
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_logf(x) log2f(x)
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __builtin_amdgcn_s_setprio(x) ((void)0)
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_wave_barrier() emu::wave_sync()
#define __builtin_amdgcn_global_load_lds(g, l, size, off, aux) \
    __builtin_memcpy((char*)(l) + (size) * emu::lane_id(), (const char*)(g), (size))
// the wave-wide effect of a wait (all lanes' copies into LDS have landed) needs a rendezvous of the lanes here
#define __builtin_amdgcn_s_waitcnt(x) emu::wave_sync()
#define __builtin_amdgcn_s_setprio(x) ((void)0)
#define __builtin_amdgcn_fence(order, scope) ((void)0)
#define hipFuncAttributeMaxDynamicSharedMemorySize 0
template <typename F>
inline hipError_t hipFuncSetAttribute(F, int, int) { return hipSuccess; }
#define __builtin_amdgcn_readfirstlane(x) (x)
#define __builtin_amdgcn_readlane(x, l) __shfl((x), (l))
#define __builtin_nontemporal_store(v, p) (*(p) = (v))
#define __builtin_nontemporal_load(p) (*(p))

template <typename T>
inline T atomicAdd(T* p, T v) { T o = *p; *p = o + v; return o; }
template <typename T>
inline T atomicOr(T* p, T v) { T o = *p; *p = o | v; return o; }
template <typename T>
inline T atomicMax(T* p, T v) { T o = *p; *p = o > v ? o : v; return o; }
template <typename T>
inline T atomicExch(T* p, T v) { T o = *p; *p = v; return o; }
inline void __threadfence() {}
inline unsigned __float_as_uint(float f) { unsigned u; memcpy(&u, &f, 4); return u; }
inline float __uint_as_float(unsigned u) { float f; memcpy(&f, &u, 4); return f; }
inline float __expf(float x) { return expf(x); }
inline float __logf(float x) { return logf(x); }
inline float rsqrtf(float x) { return 1.0f / sqrtf(x); }
template <typename T> inline T min(T a, T b) { return a < b ? a : b; }
template <typename T> inline T max(T a, T b) { return a > b ? a : b; }
