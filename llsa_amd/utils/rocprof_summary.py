"""Reduces the rocprofv3 databases of five profiled bench runs to the three text tables kept under profiles/.

    python -m llsa_amd.utils.rocprof_summary <workload> <raw directory> [<output directory>]

The raw directory holds what the commands quoted at the top of each table wrote with `-d <raw>/<name>`:
kt/t_results.db + kt.log (kernel trace and the bench line of that run), fetch/p_results.db, write/p_results.db
(FETCH_SIZE / WRITE_SIZE with the calibration copy), sq/p_results.db and cache/p_results.db (wave-scheduler and
cache counters).  Nothing here touches a GPU: the tables are averages over the dispatches in those databases."""
import sqlite3, sys, os, json
if len(sys.argv) < 3:
    sys.exit(__doc__)
wl = sys.argv[1]
desc = {'c3': 'llsa_l2 fwd+bwd B=2 H=6 N=16384 D=64 topk 16/16 RoPE in-kernel', 'c2': 'llsa_l1 fwd+bwd B=4 H=6 N=4096 D=64 topk 16',
        'n65536': 'llsa_l2 fwd+bwd B=1 H=6 N=65536 D=64 topk 16/16 RoPE in-kernel', 'c5': 'llsa_l2 fwd+bwd B=1 H=6 N=262144 D=64 topk 16/16 RoPE in-kernel',
        'c5_l3': 'llsa_l3 (three pooled levels) fwd+bwd B=1 H=6 N=262144 D=64 topk 16/16/16 RoPE in-kernel'}[wl]
raw = sys.argv[2]
out = sys.argv[3] if len(sys.argv) > 3 else os.path.join(os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))), 'profiles')
os.makedirs(out, exist_ok=True)
bench = f'python3 bench.py --workload {wl} --no-extras'

def short(n):
    n = n.replace('void ', '')
    if n.startswith('_ZN4llsa21pool_bwd_accum'): n = 'llsa::pool_bwd_accum_kernel'
    return n.split('(')[0][:60]

def durations(db):
    c = sqlite3.connect(db)
    return c.execute("select name, count(*), avg(end-start), min(end-start), max(end-start), sum(end-start) from kernels group by name order by sum(end-start) desc").fetchall()

def counters(db):
    """per (kernel, grid size): counter averages and (average duration, dispatches)"""
    c = sqlite3.connect(db)
    d, dur = {}, {}
    for k, g, n, v, a, cnt in c.execute("select kernel_name, grid_size, counter_name, avg(value), avg(duration), count(*) from counters_collection group by kernel_name, grid_size, counter_name"):
        d.setdefault((k, g), {})[n] = v
        dur[(k, g)] = (a, cnt)
    return d, dur

# ---- kernel trace
rows = durations(f'{raw}/kt/t_results.db')
line = [l for l in open(f'{raw}/kt.log') if l.startswith('{')][-1]
j = json.loads(line)
tot = sum(r[5] for r in rows)
steps = [r[1] for r in rows if 'attn_kside_kernel' in r[0]][0]      # one fine K-side launch per step
with open(f'{out}/step_kernels_{wl}_kernel_trace.txt', 'w') as f:
    f.write(f"Kernel trace of one bench run, workload {wl}: {desc}\n")
    f.write(f"command (from the repository root, on the MI355X box):\n  rocprofv3 --kernel-trace --stats -d prof/kt -o t -- {bench} --steps 20 --warmup 5\n")
    f.write(f"bench line of that run: ms_per_step={j['ms_per_step']:.4f} (under the profiler), value={j['value']:.1f} {j['unit']}\n")
    f.write(f"{steps} steps in the run (a quarter of a second untimed, 5 warm-up, 20 timed, 50 timed one by one with events); per-kernel statistics over all dispatches, durations in microseconds\n\n")
    f.write(f"{'kernel':62s} {'calls':>6s} {'avg_us':>9s} {'min_us':>9s} {'max_us':>9s} {'us/step':>9s} {'pct':>6s}\n")
    for n, cnt, a, mn, mx, s in rows:
        f.write(f"{short(n):62s} {cnt:6d} {a/1e3:9.1f} {mn/1e3:9.1f} {mx/1e3:9.1f} {s/1e3/steps:9.1f} {100*s/tot:6.1f}\n")
    f.write(f"\nsum of kernel time per step: {tot/1e3/steps:.1f} us\n")
    if wl in ('c2', 'c3'):
        f.write("(up to N = 16384 every kernel runs on the one stream: the index transposes of all levels are one launch,\n"
                " transpose_bitmap_kernel, behind the forward attention kernel)\n")
    else:
        f.write("(the index transposes -- transpose_indices_kernel, tr_*_kernel, sort_segments_kernel, inverse_positions_kernel, and\n"
                " transpose_bitmap_kernel for the pooled levels -- run on a second stream beside the forward attention kernel: their\n"
                " durations overlap with it and are stretched by it, so the sum exceeds the step time)\n")

# ---- HBM traffic
fd, fdur = counters(f'{raw}/fetch/p_results.db')
wd, wdur = counters(f'{raw}/write/p_results.db')
copyk = [k for k in fd if 'elementwise' in k[0] and fd[k]['FETCH_SIZE'] > 1e4][0]
f_fac = 262144.0 / fd[copyk]['FETCH_SIZE']
w_fac = 262144.0 / wd[copyk]['WRITE_SIZE']
with open(f'{out}/step_kernels_{wl}_hbm_traffic.txt', 'w') as f:
    f.write(f"HBM-side traffic per dispatch (L2 <-> fabric), workload {wl}: {desc}\n")
    f.write("commands (from the repository root, on the MI355X box), one counter per run:\n")
    f.write(f"  rocprofv3 --pmc FETCH_SIZE --kernel-trace -d prof/fetch -o p -- {bench} --steps 5 --warmup 2 --calibrate\n")
    f.write(f"  rocprofv3 --pmc WRITE_SIZE --kernel-trace -d prof/write -o p -- {bench} --steps 5 --warmup 2 --calibrate\n")
    f.write("--calibrate adds a plain elementwise copy of 256 MiB (torch.mul(src, 1.0, out=dst), fp32: reads 262144 KiB, writes 262144 KiB).\n")
    f.write(f"That copy reads FETCH_SIZE={fd[copyk]['FETCH_SIZE']:.0f} KiB and WRITE_SIZE={wd[copyk]['WRITE_SIZE']:.0f} KiB per dispatch, so\n")
    f.write(f"scale factors: fetch x{f_fac:.3f}, write x{w_fac:.3f}.  Values below are averages per dispatch over all dispatches of the kernel.\n\n")
    f.write("A kernel launched with several grids (the pooling pass of three levels, the reductions) has one row per grid (threads).\n\n")
    f.write(f"{'kernel':62s} {'grid':>9s} {'avg_us':>8s} {'FETCH_KiB':>10s} {'WRITE_KiB':>10s} {'read_MB':>9s} {'write_MB':>9s} {'GB/s':>8s}\n")
    traffic = {}
    for k in sorted(fd, key=lambda k: -fdur[k][0] * fdur[k][1]):
        if 'elementwise' in k[0] and k != copyk: continue
        fe, wr = fd[k]['FETCH_SIZE'], wd.get(k, {}).get('WRITE_SIZE', 0.0)
        rb, wb = fe * 1024 * f_fac, wr * 1024 * w_fac
        us = fdur[k][0] / 1e3
        f.write(f"{short(k[0]):62s} {k[1]:9d} {us:8.1f} {fe:10.0f} {wr:10.0f} {rb/1e6:9.1f} {wb/1e6:9.1f} {(rb+wb)/us/1e3:8.0f}\n")
        traffic.setdefault(short(k[0]), int(rb + wb))
    f.write("\n(read_MB / write_MB are the scaled values in 10^6 bytes; GB/s = (read + write) / avg duration)\n")
print(json.dumps(traffic, indent=1))

# ---- SQ + cache counters
sd, sdur = counters(f'{raw}/sq/p_results.db')
cd, cdur = counters(f'{raw}/cache/p_results.db')
with open(f'{out}/step_kernels_{wl}_sq_cache_counters.txt', 'w') as f:
    f.write(f"Wave-scheduler and cache counters per dispatch, workload {wl}: {desc}\n")
    f.write("commands (from the repository root, on the MI355X box):\n")
    f.write(f"  rocprofv3 --pmc SQ_WAVE_CYCLES SQ_BUSY_CU_CYCLES SQ_ACTIVE_INST_VALU SQ_ACTIVE_INST_SCA SQ_ACTIVE_INST_LDS SQ_WAIT_INST_ANY SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_VALU --kernel-trace -d prof/sq -o p -- {bench} --steps 5 --warmup 2\n")
    f.write(f"  rocprofv3 --pmc TCC_HIT_sum TCC_MISS_sum TCP_TOTAL_CACHE_ACCESSES_sum TCP_TCC_READ_REQ_sum --kernel-trace -d prof/cache -o p -- {bench} --steps 5 --warmup 2\n")
    f.write("averages per dispatch, summed over the chip.  WAVE_CYCLES, ACTIVE_INST_*, WAIT_INST_ANY are in units of 4 cycles per wave;\n")
    f.write("BUSY_CU_CYCLES and VALU_MFMA_BUSY_CYCLES in cycles.  mfma% = VALU_MFMA_BUSY_CYCLES / (duration x 2.4 GHz x 1024 SIMDs);\n")
    f.write("valu% = 4 x ACTIVE_INST_VALU / (same); wait% = WAIT_INST_ANY / WAVE_CYCLES; waves/CU = 4 x WAVE_CYCLES / (duration x 2.4 GHz x 256).\n\n")
    f.write(f"{'kernel':44s} {'grid':>9s} {'avg_us':>7s} {'mfma%':>6s} {'valu%':>6s} {'wait%':>6s} {'waves/CU':>8s} {'INSTS_VALU':>11s} {'INST_SCA':>10s} {'INST_LDS':>10s} {'L2hit%':>7s} {'TCP_acc':>10s} {'TCP->L2 rd':>10s}\n")
    for k in sorted(sd, key=lambda k: -sdur[k][0] * sdur[k][1]):
        s = sd[k]; c = cd.get(k, {})
        us = sdur[k][0] / 1e3
        simd_cyc = us * 1e-6 * 2.4e9 * 1024
        hit = c.get('TCC_HIT_sum', 0); miss = c.get('TCC_MISS_sum', 0)
        f.write(f"{short(k[0])[:44]:44s} {k[1]:9d} {us:7.1f} {100*s['SQ_VALU_MFMA_BUSY_CYCLES']/simd_cyc:6.1f} {100*4*s['SQ_ACTIVE_INST_VALU']/simd_cyc:6.1f} "
                f"{100*s['SQ_WAIT_INST_ANY']/max(s['SQ_WAVE_CYCLES'],1):6.1f} {4*s['SQ_WAVE_CYCLES']/(simd_cyc/4):8.1f} {s['SQ_INSTS_VALU']:11.3g} "
                f"{s['SQ_ACTIVE_INST_SCA']:10.3g} {s['SQ_ACTIVE_INST_LDS']:10.3g} {100*hit/max(hit+miss,1):7.1f} {c.get('TCP_TOTAL_CACHE_ACCESSES_sum',0):10.3g} {c.get('TCP_TCC_READ_REQ_sum',0):10.3g}\n")
