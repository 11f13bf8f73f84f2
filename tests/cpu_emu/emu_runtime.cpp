// Fiber scheduler behind tests/cpu_emu/include/hip/hip_runtime.h (test infrastructure).
#include <hip/hip_runtime.h>
#include <sys/mman.h>
#include <ucontext.h>
#include <vector>

namespace emu {
uint3_emu g_threadIdx, g_blockIdx;
dim3 g_blockDim, g_gridDim;

namespace {
constexpr size_t kStack = 512 * 1024;
constexpr int kWave = 64;
struct Fiber {
    ucontext_t ctx;
    bool done;
};
std::vector<Fiber> fibers;
char* stacks = nullptr;
size_t stacks_cap = 0;
ucontext_t main_ctx;
int cur = -1, nthreads = 0;
const std::function<void()>* cur_body = nullptr;
std::vector<unsigned char> smem;

// block barrier
int blk_arrived = 0;
unsigned blk_gen = 0;
// per-wave rendezvous
struct WaveSync {
    int arrived = 0;
    unsigned gen = 0;
    uint32_t stage[kWave];
    const void* ptr[kWave];
    bf16x8_t a[kWave], b[kWave];
};
std::vector<WaveSync> waves;

void yield() {
    swapcontext(&fibers[cur].ctx, &main_ctx);
}
int alive_in_wave(int w) {
    int n = 0;
    for (int i = w * kWave; i < (w + 1) * kWave && i < nthreads; i++) n += !fibers[i].done;
    return n;
}
int alive_in_block() {
    int n = 0;
    for (int i = 0; i < nthreads; i++) n += !fibers[i].done;
    return n;
}
void wave_barrier() {
    WaveSync& ws = waves[cur / kWave];
    unsigned g = ws.gen;
    ws.arrived++;
    while (ws.gen == g) {
        if (ws.arrived >= alive_in_wave(cur / kWave)) {
            ws.arrived = 0;
            ws.gen++;
            break;
        }
        yield();
    }
}
void trampoline() {
    (*cur_body)();
    fibers[cur].done = true;
    swapcontext(&fibers[cur].ctx, &main_ctx);
}
}  // namespace

int lane_id() { return cur % kWave; }
void wave_sync() { wave_barrier(); }
void* dyn_smem() { return smem.data(); }

void block_barrier() {
    unsigned g = blk_gen;
    blk_arrived++;
    while (blk_gen == g) {
        if (blk_arrived >= alive_in_block()) {
            blk_arrived = 0;
            blk_gen++;
            break;
        }
        yield();
    }
}

uint32_t shfl_u32(uint32_t v, int src_lane) {
    WaveSync& ws = waves[cur / kWave];
    ws.stage[cur % kWave] = v;
    wave_barrier();
    uint32_t r = ws.stage[src_lane & (kWave - 1)];
    wave_barrier();
    return r;
}

uint64_t ballot(bool pred) {
    WaveSync& ws = waves[cur / kWave];
    ws.stage[cur % kWave] = pred ? 1u : 0u;
    wave_barrier();
    uint64_t m = 0;
    int w = cur / kWave;
    for (int i = 0; i < kWave; i++)
        if (w * kWave + i < nthreads && !fibers[w * kWave + i].done && ws.stage[i]) m |= (1ull << i);
    wave_barrier();
    return m;
}

// D = A(16x32) * B(32x16) + C.  Lane l holds A[row l%16][k = 8*(l/16) + e], B[k = 8*(l/16) + e][col l%16]
// and D[row 4*(l/16) + e][col l%16].
f32x4_t mfma_16x16x32_bf16(bf16x8_t a, bf16x8_t b, f32x4_t c) {
    WaveSync& ws = waves[cur / kWave];
    int l = cur % kWave;
    ws.a[l] = a;
    ws.b[l] = b;
    wave_barrier();
    int col = l % 16;
    f32x4_t d = c;
    for (int e = 0; e < 4; e++) {
        int row = 4 * (l / 16) + e;
        float s = 0.f;
        for (int k = 0; k < 32; k++) {
            float av = (float)ws.a[row + 16 * (k / 8)][k % 8];
            float bv = (float)ws.b[col + 16 * (k / 8)][k % 8];
            s += av * bv;
        }
        d[e] += s;
    }
    wave_barrier();
    return d;
}

// ds_read_b64_tr_b16: in each group of 16 lanes, lane i gets element i%4 of the 8-byte chunks
// addressed by lanes i/4, 4 + i/4, 8 + i/4, 12 + i/4 (behaviour observed on gfx950 hardware).
s16x4_t ds_read_tr16_b64(const void* p) {
    WaveSync& ws = waves[cur / kWave];
    const int l = cur % kWave;
    ws.ptr[l] = p;
    wave_barrier();
    const int grp = l & ~15, i = l & 15;
    s16x4_t r;
    for (int e = 0; e < 4; e++) r[e] = reinterpret_cast<const short*>(ws.ptr[grp + 4 * e + i / 4])[i % 4];
    wave_barrier();
    return r;
}

void launch(dim3 grid, dim3 block, size_t shmem, const std::function<void()>& body) {
    nthreads = (int)(block.x * block.y * block.z);
    if (nthreads <= 0 || nthreads > 1024) {
        fprintf(stderr, "emu: bad block size %d\n", nthreads);
        abort();
    }
    if ((size_t)nthreads * kStack > stacks_cap) {
        if (stacks) munmap(stacks, stacks_cap);
        stacks_cap = (size_t)nthreads * kStack;
        stacks = (char*)mmap(nullptr, stacks_cap, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
        if (stacks == MAP_FAILED) abort();
    }
    smem.assign(shmem + 64, 0);
    g_blockDim = block;
    g_gridDim = grid;
    cur_body = &body;
    fibers.resize(nthreads);
    waves.assign((nthreads + kWave - 1) / kWave, WaveSync());
    for (unsigned bz = 0; bz < grid.z; bz++)
        for (unsigned by = 0; by < grid.y; by++)
            for (unsigned bx = 0; bx < grid.x; bx++) {
                blk_arrived = 0;
                for (auto& w : waves) w.arrived = 0;
                for (int t = 0; t < nthreads; t++) {
                    Fiber& f = fibers[t];
                    f.done = false;
                    getcontext(&f.ctx);
                    f.ctx.uc_stack.ss_sp = stacks + (size_t)t * kStack;
                    f.ctx.uc_stack.ss_size = kStack;
                    f.ctx.uc_link = &main_ctx;
                    makecontext(&f.ctx, trampoline, 0);
                }
                int remaining = nthreads;
                while (remaining > 0) {
                    remaining = 0;
                    for (int t = 0; t < nthreads; t++) {
                        if (fibers[t].done) continue;
                        cur = t;
                        g_blockIdx = {bx, by, bz};
                        g_threadIdx = {(unsigned)t % block.x, ((unsigned)t / block.x) % block.y,
                                       (unsigned)t / (block.x * block.y)};
                        swapcontext(&main_ctx, &fibers[t].ctx);
                        if (!fibers[t].done) remaining++;
                    }
                }
            }
    cur = -1;
}
}  // namespace emu
