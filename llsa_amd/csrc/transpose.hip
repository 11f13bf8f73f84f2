// Index transpose: query-major top-k lists -> key-major CSR (offsets + flat list), used by
// the dK/dV passes.  One workgroup per (b,h) does the whole counting sort in LDS:
// histogram (LDS atomics), exclusive scan, scatter with an LDS cursor, and finally every
// segment is put in ascending query-block order with a per-wave bitmap (set one bit per
// entry, then read the bits back in order), which makes the result -- and therefore the
// accumulation order of dK/dV -- independent of atomic timing.
#include "llsa_device.h"
#include "llsa_host.h"
#include "../../include/llsa_hip.h"
#include <algorithm>

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

constexpr int kTrPart = 16 * kTrThreads;       // entries per workgroup of the split path

// The middle step of every form of the transpose: counts per key block -> offsets, segment starts and the work list.
// count_of(i): entries of key block i; set_start(i, start): where the caller wants the start of segment i (its cursor);
// wave_tot: 5 * kTrWaves ints of LDS.  Called by all kTrThreads threads of the workgroup; `work` already points at the
// (b,h)'s list (or is nullptr).  E: the sum of all counts.  write_out = false: only set_start is called, offsets and work list
// stay untouched (a workgroup that shares the (b,h) with others and leaves these writes to one of them).
template <typename CountFn, typename StartFn>
__device__ __forceinline__ int offsets_and_work_list(CountFn count_of, StartFn set_start, int* wave_tot, int* __restrict__ offsets,
                                                      int* __restrict__ work, int Kb, int E_items, int E_total, int chunk,
                                                      bool write_out = true) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // exclusive scan over the counts: each thread owns `per` consecutive counters
    const int per = (Kb + kTrThreads - 1) / kTrThreads;
    const int c0 = min(tid * per, Kb), c1 = min(c0 + per, Kb);
    // l_items: short items, l_long: long items (more than chunk/2 entries)
    const int long_min = chunk / 2 + 1;
    int local = 0, l_items = 0, l_slots = 0, l_multi = 0, l_long = 0;
    for (int i = c0; i < c1; i++) {
        const int c = count_of(i);
        const int nch = max(1, (c + chunk - 1) / chunk);
        const int n_long = (nch - 1) + ((c - (nch - 1) * chunk >= long_min) ? 1 : 0);   // all chunks but the last are full
        local += c;
        l_long += n_long;
        l_items += nch - n_long;
        l_slots += (nch > 1) ? nch : 0;
        l_multi += (nch > 1) ? 1 : 0;
    }
    const int incl = wave_incl_scan(local, lane);
    const int incl_i = wave_incl_scan(l_items, lane);
    const int incl_s = wave_incl_scan(l_slots, lane);
    const int incl_m = wave_incl_scan(l_multi, lane);
    const int incl_l = wave_incl_scan(l_long, lane);
    if (lane == kWave - 1) {
        wave_tot[wave] = incl;
        wave_tot[kTrWaves + wave] = incl_i;
        wave_tot[2 * kTrWaves + wave] = incl_s;
        wave_tot[3 * kTrWaves + wave] = incl_m;
        wave_tot[4 * kTrWaves + wave] = incl_l;
    }
    __syncthreads();
    int run = incl - local, run_i = incl_i - l_items, run_s = incl_s - l_slots, run_m = incl_m - l_multi, run_l = incl_l - l_long;
    int total_long = 0;
    for (int w = 0; w < kTrWaves; w++) {
        total_long += wave_tot[4 * kTrWaves + w];
        if (w < wave) {
            run += wave_tot[w];
            run_i += wave_tot[kTrWaves + w];
            run_s += wave_tot[2 * kTrWaves + w];
            run_m += wave_tot[3 * kTrWaves + w];
            run_l += wave_tot[4 * kTrWaves + w];
        }
    }
    run_i += total_long;                                      // short items follow the long ones
    const int max_items = E_items / chunk + Kb;
    for (int i = c0; i < c1; i++) {
        const int c = count_of(i);
        if (write_out) offsets[i] = run;
        set_start(i, run);
        run += c;
        if (work != nullptr && write_out) {
            const int nch = max(1, (c + chunk - 1) / chunk);
            for (int ci = 0; ci < nch; ci++) {
                const int n_ent = min(chunk, c - ci * chunk);
                int* it = work + 4 + 4 * ((n_ent >= long_min) ? run_l++ : run_i++);
                it[0] = i;
                it[1] = run - c + ci * chunk;                  // (run already points past this segment)
                it[2] = n_ent;
                it[3] = (nch > 1) ? run_s + ci : -1;
            }
            if (nch > 1) {
                int* m = work + 4 + 4 * max_items + 4 * run_m++;
                m[0] = i;
                m[1] = run_s;
                m[2] = nch;
                m[3] = 0;
            }
            run_s += (nch > 1) ? nch : 0;
        }
    }
    if (write_out && tid == kTrThreads - 1) offsets[Kb] = run;        // (the last thread's running sum is the total)
    if (write_out && work != nullptr && tid == kTrThreads - 1) {
        work[0] = run_i;                                      // (the last thread's short items end the list)
        work[1] = run_s;
        work[2] = run_m;
        work[3] = 0;
    }
    (void)E_total;
    return run;                                               // the end of this thread's key blocks: the total for the last thread
}

// Work list (optional): the K-side kernels walk each key block's segment in chunks of at most
// `chunk` entries so that a popular key block does not serialise on one wave.  Per (b,h), all
// records 4 ints (16-byte aligned when the list is, so that one load fetches a record):
//   work[0] = number of items, work[1] = number of partial-sum slots, work[2] = number of key
//   blocks with more than one chunk, work[3] unused,
//   work[4 + 4i ..]             item i = {key block n, first entry in flat, entries, partial-sum slot
//                               or -1 when n has one chunk}      (items of one key block are adjacent),
//   work[4 + 4 max_items + 4j ..] j-th key block with more than one chunk = {n, first slot, chunks, 0}.
// Every key block has at least one item (an unselected block's item has no entries and only
// writes zeros), and max_items = Mb*T/chunk + Kb.  Items with more than chunk/2 entries come first
// in the list: a wave walks its item serially, so the long ones have to start early or the kernel
// ends with a few waves still working.
// SPLIT = false: the whole job of one (b,h).  SPLIT = true (many entries): the middle step of three --
// tr_count_kernel has left the histogram in the tail of the work list, this kernel scans it, writes
// offsets and work list and leaves every segment's start in the same place as the cursor that
// tr_scatter_kernel advances.
template <bool SPLIT>
__global__ __launch_bounds__(kTrThreads) void transpose_indices_kernel(const int* __restrict__ idx, int* __restrict__ offsets,
                                                                      int* __restrict__ flat, int* __restrict__ work,
                                                                      int Mb, int Kb, int T, int chunk, int work_stride) {
    // These kernels run beside the forward attention kernel on a second stream and are on the
    // critical path of nothing until the backward starts, but one slow workgroup per (b,h) is all
    // there is of them: let their waves go first when they share a CU.
    __builtin_amdgcn_s_setprio(3);
    HIP_DYNAMIC_SHARED(int, smem)
    int* pos = smem;                               // Kb
    int* wave_tot = smem + (SPLIT ? 0 : Kb);       // 5 * kTrWaves (the split form keeps no counters in LDS)

    const int tid = threadIdx.x;
    const int bh = blockIdx.x;
    const int E = Mb * T;
    idx += (int64_t)bh * E;
    flat += (int64_t)bh * E;
    offsets += (int64_t)bh * (Kb + 1);

    constexpr int kBatch = 16;
    int* tail = SPLIT ? work + (int64_t)bh * work_stride + (work_stride - work_tail_len(Kb)) : nullptr;
    if (!SPLIT) {
        for (int i = tid; i < Kb; i += kTrThreads) pos[i] = 0;
    }
    __syncthreads();
    // entries are taken 16 per thread at a time, all 16 loads issued before the first is used
    for (int e0 = 0; e0 < (SPLIT ? 0 : E); e0 += kBatch * kTrThreads) {
        int v[kBatch];
#pragma unroll
        for (int k = 0; k < kBatch; k++) {
            const int e = e0 + k * kTrThreads + tid;
            v[k] = (e < E) ? idx[e] : -1;
        }
#pragma unroll
        for (int k = 0; k < kBatch; k++)
            if (e0 + k * kTrThreads + tid < E) atomicAdd(&pos[clampi(v[k], 0, Kb - 1)], 1);
    }
    __syncthreads();

    if (work != nullptr) work += (int64_t)bh * work_stride;
    offsets_and_work_list([&](int i) { return SPLIT ? tail[i] : pos[i]; },
                          [&](int i, int start) {
                              if (SPLIT) tail[i] = start;
                              else pos[i] = start;
                          },
                          wave_tot, offsets, work, Kb, E, E, chunk);
    __syncthreads();

    for (int e0 = 0; e0 < (SPLIT ? 0 : E); e0 += kBatch * kTrThreads) {
        int v[kBatch];
#pragma unroll
        for (int k = 0; k < kBatch; k++) {
            const int e = e0 + k * kTrThreads + tid;
            v[k] = (e < E) ? idx[e] : -1;
        }
#pragma unroll
        for (int k = 0; k < kBatch; k++) {
            const int e = e0 + k * kTrThreads + tid;
            if (e < E) flat[atomicAdd(&pos[clampi(v[k], 0, Kb - 1)], 1)] = e / T;
        }
    }
    // pos[n] is now the END of segment n; the segments are sorted by sort_segments_kernel
}

// The whole transpose of a small job in one workgroup and one pass, sorted as it is built: the workgroup keeps one
// bitmap over the query blocks per key block in LDS (Kb rows of Mb bits; one word of padding per row keeps the rows
// off each other's banks), every entry sets its bit, a key block's count is the population of its row, and its
// segment is written by reading the row's bits back in order -- ascending query blocks with no scatter through
// atomic cursors and no sorting pass afterwards; the inverse position of an entry is its segment's start plus the
// bits below its own.  Several jobs (the selections of all levels of one operator call) share a launch:
// blockIdx.y picks the job.  A job fits when its bitmaps do (tr_bitmap_lds_ints); bigger ones take the kernels above.
// Writing the segments is the long phase (4-byte stores, every lane into a line of its own, which one CU's memory
// pipeline takes a lane at a time): a job with many key blocks is given `parts` workgroups per (b,h), each of which
// builds the same bitmaps, counts and starts for itself (cheap, and no word has to pass between workgroups) and writes
// the segments of its share of the key blocks; the first of them also writes offsets and work list.
struct TrJob {
    const int* idx; int* offsets; int* flat; int* work; int* inv;
    int Mb, Kb, T, chunk, work_stride, parts;
};
struct TrJobs {
    TrJob job[LLSA_MAX_LEVELS];
    int max_parts;                                            // workgroups per (b,h) in the grid; job i uses the first job[i].parts
};
__host__ __device__ inline int64_t tr_bitmap_lds_ints(int Mb, int Kb) { return (int64_t)Kb * ((Mb + 31) / 32 + 1) + 5 * kTrWaves; }
constexpr int64_t kTrBitmapMaxInts = 36 * 1024;               // 144 KB

__global__ __launch_bounds__(kTrThreads) void transpose_bitmap_kernel(TrJobs jobs) {
    HIP_DYNAMIC_SHARED(int, smem)
    const TrJob& jb = jobs.job[blockIdx.y];
    const int part = blockIdx.x % jobs.max_parts, bh = blockIdx.x / jobs.max_parts;
    if (part >= jb.parts) return;
    const int Mb = jb.Mb, Kb = jb.Kb, T = jb.T;
    const int words = (Mb + 31) / 32, stride = words + 1;
    unsigned* bm = reinterpret_cast<unsigned*>(smem);         // [Kb][stride]
    int* wave_tot = smem + Kb * stride;                       // 5 * kTrWaves
    const int tid = threadIdx.x;
    const int E = Mb * T;
    const int* idx = jb.idx + (int64_t)bh * E;
    int* flat = jb.flat + (int64_t)bh * E;
    int* offsets = jb.offsets + (int64_t)bh * (Kb + 1);
    int* work = jb.work ? jb.work + (int64_t)bh * jb.work_stride : nullptr;

    for (int i = tid; i < Kb * stride; i += kTrThreads) bm[i] = 0u;
    __syncthreads();
    constexpr int kBatch = 16;
    for (int e0 = 0; e0 < E; e0 += kBatch * kTrThreads) {     // 16 loads in flight per thread
        int v[kBatch];
#pragma unroll
        for (int k = 0; k < kBatch; k++) {
            const int e = e0 + k * kTrThreads + tid;
            v[k] = (e < E) ? idx[e] : -1;
        }
#pragma unroll
        for (int k = 0; k < kBatch; k++) {
            const int e = e0 + k * kTrThreads + tid;
            if (e < E) {
                const int q = e / T;
                atomicOr(&bm[clampi(v[k], 0, Kb - 1) * stride + (q >> 5)], 1u << (q & 31));
            }
        }
    }
    __syncthreads();
    // counts -> the padding word of each row; the scan then leaves the segment's start there
    for (int n = tid; n < Kb; n += kTrThreads) {
        int c = 0;
        for (int w = 0; w < words; w++) c += __popc(bm[n * stride + w]);
        bm[n * stride + words] = (unsigned)c;
    }
    __syncthreads();
    offsets_and_work_list([&](int i) { return (int)bm[i * stride + words]; },
                          [&](int i, int st) { bm[i * stride + words] = (unsigned)st; },      // the count gives way to the start
                          wave_tot, offsets, work, Kb, E, E, jb.chunk, part == 0);
    __syncthreads();                                          // (every row's start is in place)
    if (jb.inv != nullptr) {
        int* inv = jb.inv + (int64_t)bh * E;
        for (int e = part * kTrThreads + tid; e < E; e += jb.parts * kTrThreads) {
            const int q = e / T, n = clampi(idx[e], 0, Kb - 1);
            const unsigned* row = bm + n * stride;
            int pos = (int)row[words];
            for (int w = 0; w < (q >> 5); w++) pos += __popc(row[w]);
            pos += __popc(row[q >> 5] & ((1u << (q & 31)) - 1u));
            inv[e] = pos;
        }
    }
    // The segments, ascending.  Eight neighbouring lanes share a key block's row, each with an eighth of its words: the lanes
    // count their bits, a scan over the eight gives each its place in the segment, and each writes the query blocks of its
    // own words.  (One lane per row made a wave walk as many rounds as its longest segment has entries, every round a 4-byte
    // store per lane into a line of its own; this way a round writes eight segments, and a row of 16 entries takes 2 or 3.)
    const int rows = (Kb + jb.parts - 1) / jb.parts, r1 = min(Kb, (part + 1) * rows);
    const int sub = tid & 7, wps = (words + 7) / 8, w_lo = min(words, sub * wps), w_hi = min(words, w_lo + wps);
    for (int n0 = part * rows; n0 < r1; n0 += kTrThreads / 8) {
        const int n = n0 + (tid >> 3);
        const unsigned* row = bm + min(n, Kb - 1) * stride;
        int mine = 0;
        if (n < r1)
            for (int w = w_lo; w < w_hi; w++) mine += __popc(row[w]);
        int incl = mine;                                      // (all lanes take part in the shuffles)
#pragma unroll
        for (int d = 1; d < 8; d <<= 1) {
            const int o = __shfl_up(incl, d, 8);
            if (sub >= d) incl += o;
        }
        if (n >= r1) continue;
        int out = (int)row[words] + incl - mine;
        for (int w = w_lo; w < w_hi; w++) {
            unsigned wd = row[w];
            while (wd) {
                flat[out++] = w * 32 + __ffs((int)wd) - 1;
                wd &= wd - 1u;
            }
        }
    }
}

// Split path, first and last step: one workgroup per kTrPart entries.
__global__ __launch_bounds__(kTrThreads) void tr_zero_kernel(int* __restrict__ work, int Kb, int work_stride) {
    int* tail = work + (int64_t)blockIdx.x * work_stride + (work_stride - work_tail_len(Kb));
    for (int i = threadIdx.x; i < Kb; i += kTrThreads) tail[i] = 0;
}
__global__ __launch_bounds__(kTrThreads) void tr_count_kernel(const int* __restrict__ idx, int* __restrict__ work, int E, int Kb,
                                                             int work_stride) {
    // (global atomics, no LDS histogram: this kernel runs beside the forward attention kernel, whose
    // workgroups leave no room for 64 KB of LDS, and its workgroups would wait for that kernel to end)
    __builtin_amdgcn_s_setprio(3);
    const int tid = threadIdx.x, bh = blockIdx.y;
    int* tail = work + (int64_t)bh * work_stride + (work_stride - work_tail_len(Kb));
    idx += (int64_t)bh * E;
    int v[16];
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const int e = blockIdx.x * kTrPart + k * kTrThreads + tid;
        v[k] = (e < E) ? idx[e] : -1;
    }
#pragma unroll
    for (int k = 0; k < 16; k++)
        if (blockIdx.x * kTrPart + k * kTrThreads + tid < E) atomicAdd(&tail[clampi(v[k], 0, Kb - 1)], 1);
}
__global__ __launch_bounds__(kTrThreads) void tr_scatter_kernel(const int* __restrict__ idx, int* __restrict__ flat,
                                                               int* __restrict__ work, int E, int Kb, int T, int work_stride) {
    __builtin_amdgcn_s_setprio(3);
    const int tid = threadIdx.x, bh = blockIdx.y;
    int* cursor = work + (int64_t)bh * work_stride + (work_stride - work_tail_len(Kb));
    idx += (int64_t)bh * E;
    flat += (int64_t)bh * E;
    int v[16];
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const int e = blockIdx.x * kTrPart + k * kTrThreads + tid;
        v[k] = (e < E) ? idx[e] : -1;
    }
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const int e = blockIdx.x * kTrPart + k * kTrThreads + tid;
        if (e < E) flat[atomicAdd(&cursor[clampi(v[k], 0, Kb - 1)], 1)] = e / T;      // order inside a segment: sorted afterwards
    }
}

// Puts every segment of `flat` in ascending order: one wave per key block sets one bit per
// entry in a private LDS bitmap over the query blocks and reads the bits back in order.  Only the
// words between the smallest and the largest query block of the segment are cleared and read.
__global__ __launch_bounds__(256) void sort_segments_kernel(const int* __restrict__ offsets, int* __restrict__ flat, int Mb,
                                                            int Kb, int T) {
    __builtin_amdgcn_s_setprio(3);
    HIP_DYNAMIC_SHARED(unsigned, bitmaps)                     // waves x words
    const int words = (Mb + 31) / 32;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int bh = blockIdx.y, n = blockIdx.x * (int)(blockDim.x >> 6) + wave;
    if (n >= Kb) return;                                      // no workgroup barrier below
    flat += (int64_t)bh * Mb * T;
    const int* o = offsets + (int64_t)bh * (Kb + 1) + n;
    const int s = o[0], e = o[1];
    if (e - s <= 1) return;
    int qlo = Mb - 1, qhi = 0;
    for (int i = s + lane; i < e; i += kWave) {
        const int q = clampi(flat[i], 0, Mb - 1);
        qlo = q < qlo ? q : qlo;
        qhi = q > qhi ? q : qhi;
    }
    for (int d = 1; d < kWave; d <<= 1) {
        const int a = __shfl_xor(qlo, d), b = __shfl_xor(qhi, d);
        qlo = a < qlo ? a : qlo;
        qhi = b > qhi ? b : qhi;
    }
    const int w_lo = qlo >> 5, w_hi = (qhi >> 5) + 1;         // the same in every lane
    unsigned* bm = bitmaps + wave * words;
    for (int w = w_lo + lane; w < w_hi; w += kWave) bm[w] = 0u;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    for (int i = s + lane; i < e; i += kWave) {
        const int q = clampi(flat[i], 0, Mb - 1);
        atomicOr(&bm[q >> 5], 1u << (q & 31));
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    int out = s;
    for (int wb = w_lo; wb < w_hi; wb += kWave) {
        unsigned wd = (wb + lane < w_hi) ? bm[wb + lane] : 0u;
        const int cnt = __popc(wd);
        const int incl2 = wave_incl_scan(cnt, lane);
        int oo = out + incl2 - cnt;
        while (wd) {
            const int bit = __ffs((int)wd) - 1;
            flat[oo++] = (wb + lane) * 32 + bit;
            wd &= wd - 1;
        }
        out += __shfl(incl2, kWave - 1);
    }
}

// The inverse of the sorted lists: entry (query block q, slot t) of idx names key block n, and q sits somewhere in
// n's ascending segment of flat -- one thread per entry finds where by bisection.  (A row that names a key block
// twice owns one position only; both slots receive it.)
__global__ __launch_bounds__(256) void inverse_positions_kernel(const int* __restrict__ idx, const int* __restrict__ offsets,
                                                                const int* __restrict__ flat, int* __restrict__ inv, int Mb, int Kb,
                                                                int T) {
    const int e = blockIdx.x * 256 + threadIdx.x, bh = blockIdx.y;
    const int E = Mb * T;
    if (e >= E) return;
    const int q = e / T;
    const int n = clampi(idx[(int64_t)bh * E + e], 0, Kb - 1);
    const int* o = offsets + (int64_t)bh * (Kb + 1) + n;
    const int* f = flat + (int64_t)bh * E;
    int lo = o[0], hi = o[1] - 1;                             // the segment holds q: it is never empty
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (f[mid] < q) lo = mid + 1;
        else hi = mid;
    }
    inv[(int64_t)bh * E + e] = clampi(lo, 0, E - 1);
}

}  // namespace llsa

using namespace llsa;

extern "C" int llsa_fine_chunk(int N) { return fine_chunk(N); }

extern "C" int64_t llsa_work_list_len(int Mb, int Kb, int T, int chunk) {
    if (Mb <= 0 || Kb <= 0 || T <= 0 || chunk <= 0) return -1;
    const int64_t e = (int64_t)Mb * T;
    return 4 + 4 * (e / chunk + Kb) + 4 * (e / chunk + 1) + work_tail_len(Kb);
}

static int check_transpose_job(const int32_t* idx, const int32_t* offsets, const int32_t* flat, const int32_t* work, int B, int H, int Mb, int Kb,
                               int T, int chunk) {
    LLSA_REQUIRE(idx && offsets && flat, "transpose_indices: null argument");
    LLSA_REQUIRE(B > 0 && H > 0 && Mb > 0 && Kb > 0 && T > 0, "transpose_indices: bad shape");
    LLSA_REQUIRE(work == nullptr || chunk >= 1, "transpose_indices: work list needs chunk >= 1");
    return 0;
}

// the jobs whose bitmaps fit LDS, all in one launch
static int launch_bitmap_jobs(TrJobs& jobs, int n_jobs, int B, int H, hipStream_t st) {
    int64_t ints = 0;
    for (int i = 0; i < n_jobs; i++) ints = std::max(ints, tr_bitmap_lds_ints(jobs.job[i].Mb, jobs.job[i].Kb));
    const size_t lds = sizeof(int) * (size_t)ints;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)transpose_bitmap_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(-101, "transpose_indices: cannot raise dynamic LDS to %zu bytes: %s", lds, hipGetErrorString(e));
    }
    jobs.max_parts = 1;
    for (int i = 0; i < n_jobs; i++) jobs.max_parts = std::max(jobs.max_parts, jobs.job[i].parts);
    hipLaunchKernelGGL(transpose_bitmap_kernel, dim3(B * H * jobs.max_parts, n_jobs), dim3(kTrThreads), lds, st, jobs);
    return launch_status("transpose_indices");
}

static int transpose_general(const int32_t* idx, int32_t* offsets, int32_t* flat, int32_t* work, int32_t* inv, int B, int H, int Mb, int Kb,
                             int T, int chunk, void* stream) {
    const size_t lds = sizeof(int) * ((size_t)Kb + 128);
    static_assert(5 * kTrWaves <= 128, "wave totals must fit their LDS slot");
    LLSA_REQUIRE(lds <= 160 * 1024 || (work != nullptr && (int64_t)Mb * T >= 4 * kTrPart),
                 "transpose_indices: Kb=%d needs %zu bytes of LDS (limit 163840)", Kb, lds);
    // the segment sort keeps one bitmap over the query blocks per wave: four waves a workgroup while they fit, then two, then one
    const size_t bitmap = sizeof(unsigned) * ((size_t)(Mb + 31) / 32);
    const int sort_waves = 4 * bitmap <= 160 * 1024 ? 4 : 2 * bitmap <= 160 * 1024 ? 2 : 1;
    const size_t lds_sort = bitmap * sort_waves;
    LLSA_REQUIRE(lds_sort <= 160 * 1024, "transpose_indices: Mb=%d needs %zu bytes of LDS for the segment sort (limit 163840)", Mb, lds_sort);
    const int64_t E = (int64_t)Mb * T;
    const bool split = work != nullptr && E >= 4 * kTrPart;
    if (!split && lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)transpose_indices_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return fail(-101, "transpose_indices: cannot raise dynamic LDS to %zu bytes: %s", lds, hipGetErrorString(e));
    }
    const int wl = (int)llsa_work_list_len(Mb, Kb, T, chunk);
    hipStream_t st = (hipStream_t)stream;
    if (split) {
        // many entries: histogram and scatter spread over E / kTrPart workgroups per (b,h)
        const int parts = (int)((E + kTrPart - 1) / kTrPart);
        hipLaunchKernelGGL(tr_zero_kernel, dim3(B * H), dim3(kTrThreads), 0, st, work, Kb, wl);
        hipLaunchKernelGGL(tr_count_kernel, dim3(parts, B * H), dim3(kTrThreads), 0, st, idx, work, (int)E, Kb, wl);
        hipLaunchKernelGGL(HIP_KERNEL_NAME(transpose_indices_kernel<true>), dim3(B * H), dim3(kTrThreads), sizeof(int) * 128, st, idx,
                           offsets, flat, work, Mb, Kb, T, chunk, wl);
        hipLaunchKernelGGL(tr_scatter_kernel, dim3(parts, B * H), dim3(kTrThreads), 0, st, idx, flat, work, (int)E, Kb, T, wl);
    } else {
        hipLaunchKernelGGL(HIP_KERNEL_NAME(transpose_indices_kernel<false>), dim3(B * H), dim3(kTrThreads), lds, st, idx, offsets, flat,
                           work, Mb, Kb, T, chunk, wl);
    }
    if (lds_sort > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)sort_segments_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_sort);
        if (e != hipSuccess) return fail(-101, "transpose_indices: cannot raise dynamic LDS to %zu bytes: %s", lds_sort, hipGetErrorString(e));
    }
    hipLaunchKernelGGL(sort_segments_kernel, dim3((Kb + sort_waves - 1) / sort_waves, B * H), dim3(64 * sort_waves), lds_sort,
                       (hipStream_t)stream, (const int*)offsets, flat, Mb, Kb, T);
    if (inv != nullptr)
        hipLaunchKernelGGL(inverse_positions_kernel, dim3((unsigned)((E + 255) / 256), B * H), dim3(256), 0, (hipStream_t)stream, idx,
                           (const int*)offsets, (const int*)flat, inv, Mb, Kb, T);
    return launch_status("transpose_indices");
}

extern "C" int llsa_transpose_indices_multi(const llsa_transpose_job* jobs, int n_jobs, int B, int H, void* stream) {
    LLSA_REQUIRE(jobs != nullptr && n_jobs >= 1 && n_jobs <= LLSA_MAX_LEVELS, "transpose_indices: 1..%d jobs, got %d", LLSA_MAX_LEVELS, n_jobs);
    // One launch when the bitmaps of every job fit.  Beside a job that is too large for that, a small job shares the
    // launch of the small ones only while its bitmaps are light (32 KB): a workgroup that wants most of a CU's LDS waits
    // for a CU to drain when it runs next to the large job's kernels -- or next to an attention kernel on another
    // stream, which is where a caller with large jobs runs this (0.6 ms instead of 16 us for the level-1 selection of
    // 262144 tokens beside the forward kernel) -- so such a job takes the kernels for large jobs too.
    bool all_fit = true;
    for (int i = 0; i < n_jobs; i++) {
        const llsa_transpose_job& j = jobs[i];
        const int rc = check_transpose_job(j.idx, j.offsets, j.flat, j.work, B, H, j.Mb, j.Kb, j.T, j.chunk);
        if (rc != 0) return rc;
        all_fit = all_fit && tr_bitmap_lds_ints(j.Mb, j.Kb) <= kTrBitmapMaxInts;
    }
    constexpr int64_t kLightInts = 8 * 1024;
    TrJobs small;
    int n_small = 0;
    for (int i = 0; i < n_jobs; i++) {
        const llsa_transpose_job& j = jobs[i];
        const int chunk = j.chunk < 1 ? 1 : j.chunk;
        if (tr_bitmap_lds_ints(j.Mb, j.Kb) <= (all_fit ? kTrBitmapMaxInts : kLightInts)) {
            TrJob& t = small.job[n_small++];
            t.idx = j.idx; t.offsets = j.offsets; t.flat = j.flat; t.work = j.work; t.inv = j.inv;
            t.Mb = j.Mb; t.Kb = j.Kb; t.T = j.T; t.chunk = chunk;
            t.work_stride = j.work ? (int)llsa_work_list_len(j.Mb, j.Kb, j.T, chunk) : 0;
            t.parts = std::min(8, std::max(1, j.Kb / 128));
        } else {
            const int rc = transpose_general(j.idx, j.offsets, j.flat, j.work, j.inv, B, H, j.Mb, j.Kb, j.T, chunk, stream);
            if (rc != 0) return rc;
        }
    }
    if (n_small > 0) return launch_bitmap_jobs(small, n_small, B, H, (hipStream_t)stream);
    return 0;
}

extern "C" int llsa_transpose_indices(const int32_t* idx, int32_t* offsets, int32_t* flat, int32_t* work, int32_t* inv, int B, int H,
                                      int Mb, int Kb, int T, int chunk, void* stream) {
    llsa_transpose_job j;
    j.idx = idx; j.offsets = offsets; j.flat = flat; j.work = work; j.inv = inv;
    j.Mb = Mb; j.Kb = Kb; j.T = T; j.chunk = chunk;
    return llsa_transpose_indices_multi(&j, 1, B, H, stream);
}
