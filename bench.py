#!/usr/bin/env python3
"""Benchmark of the GEMM hot path on one MI355X.

A step is one FP8 e4m3 block-scaled GEMM at M=4096, N=7168, K=7168 (per-token 1x128 activation scales, 128x128
weight scales, bf16 output) through the JIT entry point, inputs resident in HBM before the timed region.
Prints ONE JSON line: whole-job TFLOPS, the roofline position of the GEMM kernel (HIP-event time of the launches
on the stream they run on), the other baseline configurations as compact legs under `extra` (bf16 8192^3 next to
the vendor library on the same operands, the M=64 decode shape, FP8 16384^3 with outliers) and a torch-CPU baseline
of the same workload. `--also` adds the grouped GEMMs, the quantisers and the fp32 GEMM to `extra`.

Order of operations for every leg: `settle` untimed launches of the same kernel, `warmup` untimed launches, the timed
launches, and only then the validity check. The settle phase exists because the chip's power controller reacts to the
onset of a matrix-core load: coming from idle the first ~10 launches run at the steady rate, the next ~30 run up to a
third slower while the clock is pulled down, and the rate is back to steady only after ~100 launches. A run that times
25 launches after an idle period measures that transient, not the kernel. The count is printed with each leg.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, 'tests'))
os.environ.setdefault('YAN_CACHE_DIR', os.path.join(ROOT, '.yan_cache'))

METRIC = 'TFLOPS & % of MFMA peak, fp8 block-scaled GEMM 4096x7168x7168, 1 MI355X'
# MI355X vendor peaks (dense): the one place these constants live.
PEAK_FP8_TFLOPS = 5000.0
PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBPS = 8000.0
PEAK_FP32_TFLOPS = 157.3
# Untimed launches of the leg's own kernel before its warm-up: about 100 ms of load each.
SETTLE = {'cfg3': 600, 'cfg2': 150, 'cfg4': 2000, 'cfg5': 30}


def _event_time_ms(fn, steps, warmup, settle=0):
    """Average device time of one call over `steps` back-to-back calls, from events on the current stream, after
    `settle` + `warmup` untimed calls. Returns (event ms per call, wall ms per call)."""
    import torch
    for _ in range(settle):
        fn()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return start.elapsed_time(end) / steps, wall_ms / steps


def _clock_and_power(fn, seconds=0.4):
    """Shader clock (MHz) and board power (W) while `fn` is launched back to back for about `seconds`, read from the
    amdgpu driver's sysfs files (pp_dpm_sclk, hwmon power1_input / power1_average) every few milliseconds; None where
    the files are absent or unreadable. Outside every timed region: the sampling thread shares the interpreter with
    the launch loop."""
    import glob
    import threading
    import torch
    sclk = (glob.glob('/sys/class/drm/card*/device/pp_dpm_sclk') + [None])[0]
    power = (glob.glob('/sys/class/drm/card*/device/hwmon/hwmon*/power1_input') +
             glob.glob('/sys/class/drm/card*/device/hwmon/hwmon*/power1_average') + [None])[0]
    if sclk is None and power is None:
        return None
    clocks, watts, stop = [], [], threading.Event()

    def sample():
        while not stop.is_set():
            try:
                if sclk:
                    active = [line for line in open(sclk).read().splitlines() if line.rstrip().endswith('*')]
                    if active:
                        clocks.append(float(active[0].split(':')[1].lower().replace('mhz', '').replace('*', '').strip()))
                if power:
                    watts.append(float(open(power).read()) * 1e-6)
            except (OSError, ValueError, IndexError):
                pass
            time.sleep(0.004)

    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    per_call = (time.perf_counter() - t0) / 20
    calls = max(20, int(seconds / max(per_call, 1e-6)))
    for _ in range(calls // 2):         # back under load before sampling starts
        fn()
    thread = threading.Thread(target=sample, daemon=True)
    thread.start()
    for _ in range(calls):
        fn()
    torch.cuda.synchronize()
    stop.set()
    thread.join()
    mean = lambda xs: round(sum(xs) / len(xs), 1) if xs else None
    return {'shader_clock_mhz': mean(clocks), 'board_power_w': mean(watts), 'samples': max(len(clocks), len(watts))}


def _cpu_baseline_fp8(a8, sa, b8, sb, budget_s=12.0):
    """The reference's CPU path for this metric: torch CPU matmul of the dequantised operands (fp32), timed on a
    slab of rows sized for about `budget_s` seconds, scaled to the full M by the flop count."""
    import torch
    import oracle
    import harness
    m, k = a8.shape
    n = b8.shape[0]
    b_cpu, sb_cpu = b8.cpu(), sb.cpu()
    wd = harness.dequant_rhs(b_cpu, sb_cpu)

    def run(rows):
        t0 = time.perf_counter()
        x = harness.dequant_lhs(a8[:rows].cpu(), sa[:rows].cpu())
        out = x @ wd.t()
        return time.perf_counter() - t0, out

    t_probe, _ = run(32)
    t_probe, _ = run(32)
    rows = int(min(m, max(64, 32 * budget_s / max(t_probe, 1e-4) // 64 * 64)))
    reps = []
    for _ in range(2):
        t, out = run(rows)
        reps.append(t)
    t = min(reps)
    # the slab is also the oracle's check of the baseline itself
    ref = oracle.gemm_fp8_block_scaled_ref(a8[:64].view(torch.uint8).cpu().numpy(), sa[:64].cpu().numpy(),
                                           b_cpu.view(torch.uint8).numpy(), sb_cpu.numpy())
    assert oracle.calc_diff(out[:64].numpy(), ref) < 1e-9
    return {'value': round(2.0 * rows * n * k / t / 1e12, 4), 'unit': 'TFLOPS', 'cores': torch.get_num_threads(),
            'kind': 'port', 'sample': f'torch CPU fp32 matmul of dequantised operands, first {rows} of {m} rows x N={n} x K={k}, '
                                      f'best of 2, {t:.2f} s, os.cpu_count()={os.cpu_count()}'}


def _measured_traffic():
    """HBM-side bytes per launch of the GEMM kernel as measured with rocprofv3 hardware counters (FETCH_SIZE +
    WRITE_SIZE, scaled by a copy of known size). The figure is kept with the profile summary it comes from, which also
    records the digest of the kernel headers it was taken with: (bytes, digest) when that digest is the one of the
    headers in this tree, (None, digest-or-None) when the profile is absent or older than the kernel."""
    from yan_amd.jit.compiler import get_yan_version
    path = os.path.join(ROOT, 'profiles', 'fp8_gemm_4096x7168x7168_hbm_traffic.md')
    traffic = version = None
    try:
        for line in open(path):
            if line.startswith('traffic_bytes_per_launch:'):
                traffic = float(line.split(':', 1)[1].split()[0])
            elif line.startswith('kernel_headers_digest:'):
                version = line.split(':', 1)[1].split()[0]
    except OSError:
        pass
    if traffic is None or version != get_yan_version():
        return None, version
    return traffic, version


def _fp8_bytes(m, n, k):
    return m * k + n * k + 4 * m * (k // 128) + 4 * ((n + 127) // 128) * (k // 128) + 2 * m * n


def _sampled_fp8_diff(yan, harness, a8, sa, b8, sb, out, rows=256):
    import torch
    m = a8.shape[0]
    pick = torch.randperm(m, device='cuda')[:min(rows, m)]
    wd_t = harness.dequant_rhs(b8, sb).t() if b8.numel() <= (1 << 27) else None
    if wd_t is not None:
        ref = harness.dequant_lhs(a8[pick], sa[pick]) @ wd_t
    else:       # 16384^2 weights: dequantise in column slabs
        x = harness.dequant_lhs(a8[pick], sa[pick])
        ref = torch.cat([x @ harness.dequant_rhs(b8[c0:c0 + 2048], sb[c0 // 128:c0 // 128 + 16]).t()
                         for c0 in range(0, b8.shape[0], 2048)], dim=1)
    return float(yan.calc_diff(out[pick].float(), ref))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=200)
    ap.add_argument('--warmup', type=int, default=20)
    ap.add_argument('--also', action='store_true', help='also time the grouped GEMMs, the quantisers and the fp32 GEMM (more extra fields)')
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    ap.add_argument('--no-extra', action='store_true', help='skip the legs of the other baseline configurations')
    ap.add_argument('--no-settle', action='store_true', help='skip the untimed settle launches (shows the power transient)')
    ap.add_argument('--calibrate-copy', action='store_true',
                    help='also run a 1 GiB device-to-device copy three times, as the known-size kernel that hardware '
                         'byte counters (FETCH_SIZE / WRITE_SIZE) are scaled by when profiling')
    args = ap.parse_args()
    if args.gpus != 1:
        print(f'bench.py: this build runs on one GPU; --gpus {args.gpus} is not supported (every figure is a 1-GPU figure)',
              file=sys.stderr)
        sys.exit(2)

    import torch
    import yan_amd as yan
    import harness
    from yan_amd.jit_kernels.gemm import fp8_kernel_plan
    from yan_amd.jit_kernels.heuristics import get_best_dense_config
    assert torch.cuda.is_available(), 'bench.py needs a GPU'
    torch.cuda.set_device(0)
    settle = {leg: (0 if args.no_settle else count) for leg, count in SETTLE.items()}

    m, n, k = harness.BASELINE_FP8['cfg3']
    (a8, sa), (b8, sb), out = harness.make_fp8_case(m, n, k, seed=42, device='cuda', gen_device='cuda')
    sa = yan.get_col_major_tensor(sa)      # token-contiguous scales, the layout DeepGEMM-style callers hand over
    step = lambda: yan.gemm_fp8_fp8_bf16_nt((a8, sa), (b8, sb), out)
    step()                                  # loads the kernel
    torch.cuda.synchronize()

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device='cuda').fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # The same measurement without the settle phase, coming from an idle chip: what a caller gets for its first launches.
    time.sleep(0.5)
    idle_kernel_ms, idle_wall_ms = _event_time_ms(step, args.steps, args.warmup, 0)
    kernel_ms, wall_ms = _event_time_ms(step, args.steps, args.warmup, settle['cfg3'])
    # validity of what was timed: sampled rows against an fp32 matmul of the dequantised operands
    diff = _sampled_fp8_diff(yan, harness, a8, sa, b8, sb, out)
    assert diff < 1e-3, f'parity lost: calc_diff={diff}'
    under_load = _clock_and_power(step)
    flops = 2.0 * m * n * k
    tflops_job = flops / (wall_ms * 1e-3) / 1e12
    tflops_kernel = flops / (kernel_ms * 1e-3) / 1e12
    _, keys, _, _, _ = fp8_kernel_plan(m, n, k, yan.get_num_sms())
    traffic, traffic_digest = _measured_traffic()

    line = {
        'metric': METRIC, 'value': round(tflops_job, 1), 'unit': 'TFLOPS', 'n_gpus': 1,
        'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(wall_ms, 5),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'fp8_e4m3 (fp32 accumulate, bf16 out)',
        'data': 'synthetic: N(0,1) sources, seed 42, quantised per-token 1x128 / per-block 128x128',
        'config': {'workload': 'configs[2]: FP8 e4m3 block-scaled GEMM M=4096 N=7168 K=7168, bf16 out',
                   'tile': f"{keys['BLOCK_M']}x{keys['BLOCK_N']}x128", 'cache_state': 'warm (same operands every step)',
                   'settle_launches': settle['cfg3'],
                   'settle': 'untimed launches of the same kernel before the warm-up: the power controller takes ~100 launches '
                             'to settle after an idle period',
                   'tflops_from_idle': round(2.0 * m * n * k / (idle_wall_ms * 1e-3) / 1e12, 1),
                   'kernel_us_from_idle': round(idle_kernel_ms * 1e3, 2),
                   'from_idle': 'the same warm-up and timed steps after half a second of idle and no settle launches; `value` is the settled figure',
                   'calc_diff_sampled_rows': diff},
        'roofline': {'bound': 'mfma', 'achieved': round(tflops_kernel, 1), 'peak': PEAK_FP8_TFLOPS, 'unit': 'TFLOP/s',
                     'frac': round(tflops_kernel / PEAK_FP8_TFLOPS, 4), 'traffic': traffic,
                     'traffic_source': f'profiles/fp8_gemm_4096x7168x7168_hbm_traffic.md, kernel headers {traffic_digest}'
                                       if traffic is not None else 'no profile of the kernel headers in this tree',
                     'kernel': 'fp8_gemm_kernel', 'kernel_us': round(kernel_ms * 1e3, 2),
                     'algorithmic_flop_per_launch': flops, 'algorithmic_bytes_per_launch': _fp8_bytes(m, n, k)},
    }
    if under_load and under_load['shader_clock_mhz']:
        # the chip is power-limited under this load: the same kernel time as a fraction of the matrix-core cycles that
        # passed at the clock the chip actually ran at (256 CUs x 8192 flop per cycle)
        line['roofline']['under_load'] = under_load
        line['roofline']['frac_of_mfma_cycles_at_measured_clock'] = round(
            tflops_kernel * 1e12 / (yan.get_num_sms() * 8192 * under_load['shader_clock_mhz'] * 1e6), 4)

    extra = {}
    if not args.no_extra:
        # configs[1]: bf16 8192^3, next to torch.matmul (hipBLASLt) on the same operands
        mm, nn, kk = harness.BASELINE_BF16['cfg2']
        a, b, c = harness.make_bf16_case(mm, nn, kk, seed=42, scale=kk ** -0.5, device='cuda', gen_device='cuda')
        ms, _ = _event_time_ms(lambda: yan.gemm_bf16_tn(a, b, c), 20, 5, settle['cfg2'])
        pick = torch.randperm(mm, device='cuda')[:256]
        d = float(yan.calc_diff(c[pick].float(), a[pick].float() @ b.float().t()))
        assert d < 1e-5, f'bf16 parity lost: calc_diff={d}'
        fl = 2.0 * mm * nn * kk
        extra['bf16_8192'] = {'us': round(ms * 1e3, 1), 'tflops': round(fl / ms / 1e9, 1),
                              'frac_of_bf16_peak': round(fl / ms / 1e9 / PEAK_BF16_TFLOPS, 4), 'steps': 20, 'warmup': 5,
                              'settle_launches': settle['cfg2'], 'calc_diff_sampled_rows': d}
        load = _clock_and_power(lambda: yan.gemm_bf16_tn(a, b, c))
        if load and load['shader_clock_mhz']:
            extra['bf16_8192']['under_load'] = load
            extra['bf16_8192']['frac_of_mfma_cycles_at_measured_clock'] = round(
                fl / ms / 1e9 * 1e12 / (yan.get_num_sms() * 4096 * load['shader_clock_mhz'] * 1e6), 4)
        ms, _ = _event_time_ms(lambda: torch.matmul(a, b.t(), out=c), 20, 5, settle['cfg2'])
        extra['bf16_8192_torch_hipblaslt'] = {'us': round(ms * 1e3, 1), 'tflops': round(fl / ms / 1e9, 1)}
        load = _clock_and_power(lambda: torch.matmul(a, b.t(), out=c))
        if load and load['shader_clock_mhz']:
            extra['bf16_8192_torch_hipblaslt']['under_load'] = load
        del a, b, c
        # configs[3]: the M=64 decode shape, HBM-bound. The kernel is shorter than the host side of a call, so its
        # device time comes from the profiler; cold = a 512 MB write before every call.
        mm, nn, kk = harness.BASELINE_FP8['cfg4']
        (x8, sx), (w8, sw), o = harness.make_fp8_case(mm, nn, kk, seed=42, device='cuda')
        sx = yan.get_col_major_tensor(sx)
        decode = lambda: yan.gemm_fp8_fp8_bf16_nt((x8, sx), (w8, sw), o)
        _, wall = _event_time_ms(decode, 200, 20, settle['cfg4'])
        t_warm = yan.bench_kineto(decode, 'fp8_gemm', suppress_kineto_output=True)
        t_cold = yan.bench_kineto(decode, 'fp8_gemm', suppress_kineto_output=True, flush_l2=True)
        d = _sampled_fp8_diff(yan, harness, x8, sx, w8, sw, o)
        assert d < 1e-3, f'decode parity lost: calc_diff={d}'
        # The Python entry spends longer on the host than the kernel on the device, so the launches above start on an idle
        # GPU, which costs a kernel this short about 1 us. The same JIT kernels launched through their `launch` symbol with
        # prepared arguments (3 us of host work per call, the launches queue up): the split-K plan the entry uses and the
        # unsplit kernel it would use without one.
        from yan_amd import jit
        from yan_amd.jit_kernels import gemm as fp8_entry
        stream, cus = torch.cuda.current_stream(), yan.get_num_sms()
        name, keys, defs, smem, tmpl = fp8_entry.fp8_kernel_plan(mm, nn, kk, cus, True)
        unsplit = jit.build(name, defs, jit.generate(fp8_entry.includes, defs, jit.cpp_format(tmpl, keys)))
        t_unsplit = yan.bench_kineto(lambda: unsplit(x8, sx, w8, sw, o, mm, stream, cus, smem), 'fp8_gemm', suppress_kineto_output=True)
        plan, t_split = fp8_entry.fp8_split_k_plan(mm, nn, kk, cus, True), None
        if plan is not None:
            name, keys, defs, tmpl = plan
            split = jit.build(name, defs, jit.generate(fp8_entry.includes, defs, jit.cpp_format(tmpl, keys)))
            workspace, _ = fp8_entry.split_k_workspace(o.device, stream.cuda_stream)
            t_split = yan.bench_kineto(lambda: split(x8, sx, w8, sw, o, mm, stream, cus, smem, workspace, fp8_entry.SPLIT_K_WORKSPACE_BYTES),
                                       'fp8_gemm', suppress_kineto_output=True)
        # Weights from HBM, everything else warm, as a model's layers present them: every launch takes the next of enough copies
        # of the weights to exceed the caches (more than 600 MB together).
        layers = [(w8.clone(), sw.clone()) for _ in range(max(2, (600 << 20) // (nn * kk)))]
        if plan is not None:
            one_layer = lambda w, s: split(x8, sx, w, s, o, mm, stream, cus, smem, workspace, fp8_entry.SPLIT_K_WORKSPACE_BYTES)
        else:
            one_layer = lambda w, s: unsplit(x8, sx, w, s, o, mm, stream, cus, smem)
        def all_layers():
            for w, s in layers:
                one_layer(w, s)
        t_layers = yan.bench_kineto(all_layers, 'fp8_gemm', num_tests=10, suppress_kineto_output=True)
        del layers
        byt = _fp8_bytes(mm, nn, kk)
        extra['fp8_decode_64x4096x7168'] = {'kernel_us_cycling_weights': round(t_layers * 1e6, 2),
                                            'gb_per_s_cycling_weights': round(byt / t_layers / 1e9, 1),
                                            'frac_of_hbm_peak_cycling_weights': round(byt / t_layers / 1e9 / PEAK_HBM_GBPS, 4),
                                            'kernel_us_warm': round(t_warm * 1e6, 2), 'kernel_us_cold': round(t_cold * 1e6, 2),
                                            'call_to_call_us': round(wall * 1e3, 2), 'algorithmic_bytes': byt,
                                            'kernel_us_warm_queued_launches': round(t_split * 1e6, 2) if t_split else None,
                                            'kernel_us_warm_queued_launches_unsplit': round(t_unsplit * 1e6, 2),
                                            'split_k_plan': [plan[1][key] for key in ('BLOCK_M', 'BLOCK_N', 'SPLIT_K')] if plan else None,
                                            'gb_per_s_warm': round(byt / t_warm / 1e9, 1), 'gb_per_s_cold': round(byt / t_cold / 1e9, 1),
                                            'frac_of_hbm_peak_warm': round(byt / t_warm / 1e9 / PEAK_HBM_GBPS, 4),
                                            'frac_of_hbm_peak_cold': round(byt / t_cold / 1e9 / PEAK_HBM_GBPS, 4),
                                            'calc_diff': d}
        # The same decode step from bf16 activations: the quantiser and the GEMM as two entry calls, and as the one call of the
        # entry that enqueues both from one `launch` (same kernels, same bits; what differs is the host's share).
        xb = torch.randn(mm, kk, device='cuda', generator=torch.Generator(device='cuda').manual_seed(42)).bfloat16()
        two_calls = lambda: yan.gemm_fp8_fp8_bf16_nt(yan.per_token_cast_to_fp8(xb, col_major_scales=True), (w8, sw), o)
        one_call = lambda: yan.gemm_bf16_fp8_bf16_nt(xb, (w8, sw), o)
        two_calls()
        torch.cuda.synchronize()
        expect = o.clone()
        one_call()
        torch.cuda.synchronize()
        assert torch.equal(o, expect), 'the chained entry lost the bits of quantiser + GEMM'
        _, wall_two = _event_time_ms(two_calls, 500, 50, 0)
        _, wall_one = _event_time_ms(one_call, 500, 50, 0)
        t_cast = yan.bench_kineto(one_call, 'per_token_cast', suppress_kineto_output=True)
        extra['fp8_decode_64x4096x7168']['from_bf16_activations'] = {
            'call_to_call_us_quantiser_then_gemm_two_calls': round(wall_two * 1e3, 2),
            'call_to_call_us_one_call': round(wall_one * 1e3, 2), 'quantiser_kernel_us': round(t_cast * 1e6, 2), 'same_bits': True}
        del x8, sx, w8, sw, o, xb
        # configs[4]: FP8 16384^3, uniform[-4, 4] sources with 1 % of the entries x 50
        mm, nn, kk = harness.BASELINE_FP8['cfg5']
        (x8, sx), (w8, sw), o = harness.make_fp8_case(mm, nn, kk, seed=42, dist='outlier', device='cuda', gen_device='cuda')
        sx = yan.get_col_major_tensor(sx)
        ms, _ = _event_time_ms(lambda: yan.gemm_fp8_fp8_bf16_nt((x8, sx), (w8, sw), o), 10, 2, settle['cfg5'])
        d = _sampled_fp8_diff(yan, harness, x8, sx, w8, sw, o, rows=128)
        assert d < 1e-3, f'16384^3 parity lost: calc_diff={d}'
        fl = 2.0 * mm * nn * kk
        extra['fp8_16384_outliers'] = {'us': round(ms * 1e3, 1), 'tflops': round(fl / ms / 1e9, 1),
                                       'frac_of_fp8_peak': round(fl / ms / 1e9 / PEAK_FP8_TFLOPS, 4), 'steps': 10, 'warmup': 2,
                                       'settle_launches': settle['cfg5'], 'calc_diff_sampled_rows': d}
        del x8, sx, w8, sw, o

    if args.also:
        # bf16 with few rows and long K, where the entry point splits K: a decode-like shape and the m = 256 shapes of the
        # reference's own dense test with k >= 5120 (tests/test_cute.py), next to torch.matmul (hipBLASLt). Both sides cycle
        # through copies of the weights that together exceed the caches, as a model's layers do.
        from yan_amd.jit_kernels.heuristics import get_split_k_dense_config
        for mm, nn, kk in ((64, 4096, 7168), (256, 2048, 7168), (256, 5120, 5120), (256, 7168, 16384)):
            a, b, c = harness.make_bf16_case(mm, nn, kk, seed=42, scale=kk ** -0.5, device='cuda', gen_device='cuda')
            weights = [b.clone() for _ in range(min(40, max(2, (600 << 20) // (nn * kk * 2))))]
            def cycle(fn):
                def run():
                    for w in weights:
                        fn(w)
                return run
            per = len(weights)
            ms, _ = _event_time_ms(cycle(lambda w: yan.gemm_bf16_tn(a, w, c)), 8, 2, 4)
            ms_t, _ = _event_time_ms(cycle(lambda w: torch.matmul(a, w.t(), out=c)), 8, 2, 4)
            plan = get_split_k_dense_config(mm, nn, kk, yan.get_num_sms())
            extra[f'bf16_{mm}x{nn}x{kk}_cycling_weights'] = {'us': round(ms * 1e3 / per, 2), 'torch_hipblaslt_us': round(ms_t * 1e3 / per, 2),
                                                            'hipblaslt_over_this': round(ms_t / ms, 3), 'split_k_plan': list(plan) if plan else None,
                                                            'weight_copies': per}
            del a, b, c, weights
        # bf16 shapes whose tiles do not fill whole rounds of 256 compute units at 256 x 256, next to torch.matmul (hipBLASLt)
        for mm, nn, kk in ((4096, 5120, 5120), (2048, 7168, 7168), (4096, 7168, 16384), (8192, 8192, 9216)):
            a, b, c = harness.make_bf16_case(mm, nn, kk, seed=42, scale=kk ** -0.5, device='cuda', gen_device='cuda')
            ms, _ = _event_time_ms(lambda: yan.gemm_bf16_tn(a, b, c), 30, 5, 200)
            ms_t, _ = _event_time_ms(lambda: torch.matmul(a, b.t(), out=c), 30, 5, 200)
            fl = 2.0 * mm * nn * kk
            extra[f'bf16_{mm}x{nn}x{kk}'] = {'us': round(ms * 1e3, 1), 'tflops': round(fl / ms / 1e9, 1),
                                             'frac_of_bf16_peak': round(fl / ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                                             'tile': 'x'.join(map(str, get_best_dense_config(mm, nn, kk, yan.get_num_sms()))),
                                             'torch_hipblaslt_us': round(ms_t * 1e3, 1), 'hipblaslt_over_this': round(ms_t / ms, 3)}
            del a, b, c
        # grouped (mixture-of-experts) layouts: 4 groups x 8192 rows contiguous; 4 groups x 1024 of 1024 rows masked
        rows, nn, kk = (8192,) * 4, 4096, 7168
        (x8, sx), (w8, sw), o, idx = harness.make_grouped_contiguous_case(rows, nn, kk, seed=42, device='cuda', gen_device='cuda')
        sx = yan.get_col_major_tensor(sx)
        ms, _ = _event_time_ms(lambda: yan.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((x8, sx), (w8, sw), o, idx), 20, 3, 100)
        fl = 2.0 * sum(rows) * nn * kk
        extra['fp8_grouped_contiguous_4x8192x4096x7168'] = {'us': round(ms * 1e3, 1), 'tflops': round(fl / ms / 1e9, 1),
                                                            'frac_of_fp8_peak': round(fl / ms / 1e9 / PEAK_FP8_TFLOPS, 4)}
        del x8, sx, w8, sw, o, idx
        # groups whose boundaries fall in the middle of 256-row tiles (every other one): 8 groups of 896 and 1152 rows, next to
        # 8 groups of 1024 rows
        # and groups of a few hundred rows, which run the kernel that picks its tile height on the device: 256 x 256 tiles when every
        # boundary falls on a multiple of 256 rows (16 groups of 512), 128 x 256 when not (16 groups of 384 and 640)
        for label, rows in (('8x896_1152', (896, 1152) * 4), ('8x1024', (1024,) * 8), ('16x512', (512,) * 16), ('16x384_640', (384, 640) * 8)):
            (x8, sx), (w8, sw), o, idx = harness.make_grouped_contiguous_case(rows, nn, kk, seed=42, device='cuda', gen_device='cuda')
            sx = yan.get_col_major_tensor(sx)
            ms, _ = _event_time_ms(lambda: yan.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous((x8, sx), (w8, sw), o, idx), 30, 5, 150)
            fl = 2.0 * sum(rows) * nn * kk
            extra[f'fp8_grouped_contiguous_{label}x4096x7168'] = {'us': round(ms * 1e3, 1), 'tflops': round(fl / ms / 1e9, 1),
                                                                 'frac_of_fp8_peak': round(fl / ms / 1e9 / PEAK_FP8_TFLOPS, 4)}
            del x8, sx, w8, sw, o, idx
        (x8, sx), (w8, sw), o, mm_ = harness.make_grouped_masked_case(4, 1024, nn, kk, (1024,) * 4, seed=42, device='cuda', gen_device='cuda')
        sx = yan.get_col_major_tensor(sx)
        ms, _ = _event_time_ms(lambda: yan.m_grouped_gemm_fp8_fp8_bf16_nt_masked((x8, sx), (w8, sw), o, mm_, 1024), 50, 5, 600)
        fl = 2.0 * 4 * 1024 * nn * kk
        extra['fp8_grouped_masked_4x1024x4096x7168'] = {'us': round(ms * 1e3, 1), 'tflops': round(fl / ms / 1e9, 1),
                                                        'frac_of_fp8_peak': round(fl / ms / 1e9 / PEAK_FP8_TFLOPS, 4)}
        del x8, sx, w8, sw, o
        # the masked layout at decode sizes: 32 groups holding 8 rows each of 64; 940 MB of weights, more than the caches
        # hold, so every launch streams them from HBM
        groups, held = 32, 8
        (x8, sx), (w8, sw), o, mm_ = harness.make_grouped_masked_case(groups, 64, nn, kk, (held,) * groups, seed=42, device='cuda', gen_device='cuda')
        sx = yan.get_col_major_tensor(sx)
        t = yan.bench_kineto(lambda: yan.m_grouped_gemm_fp8_fp8_bf16_nt_masked((x8, sx), (w8, sw), o, mm_, held), 'fp8_gemm',
                             suppress_kineto_output=True)
        byt = groups * (nn * kk + 4 * ((nn + 127) // 128) * (kk // 128) + held * (kk + 4 * (kk // 128)) + held * nn * 2)
        extra['fp8_grouped_masked_decode_32x8x4096x7168'] = {'kernel_us': round(t * 1e6, 1), 'algorithmic_bytes': byt,
                                                             'gb_per_s': round(byt / t / 1e9, 1),
                                                             'frac_of_hbm_peak': round(byt / t / 1e9 / PEAK_HBM_GBPS, 4)}
        del x8, sx, w8, sw, o
        # quantisers in front of the GEMM (HBM-bound): cfg3's activations per token, its weights per block, from bf16
        mm, nn, kk = harness.BASELINE_FP8['cfg3']
        xs = torch.randn(mm, kk, device='cuda').bfloat16()
        ws = torch.randn(nn, kk, device='cuda').bfloat16()
        for name, fn, kern, elems, groups in (
                ('per_token_cast_4096x7168_bf16', lambda: yan.per_token_cast_to_fp8(xs, col_major_scales=True), 'per_token_cast_kernel', mm * kk, mm * kk // 128),
                ('per_block_cast_7168x7168_bf16', lambda: yan.per_block_cast_to_fp8(ws), 'per_block_cast_kernel', nn * kk, (nn // 128) * (kk // 128))):
            t_warm = yan.bench_kineto(fn, kern, suppress_kineto_output=True)
            t_cold = yan.bench_kineto(fn, kern, suppress_kineto_output=True, flush_l2=True)
            byt = 3 * elems + 4 * groups
            extra[name] = {'kernel_us_warm': round(t_warm * 1e6, 2), 'kernel_us_cold': round(t_cold * 1e6, 2),
                           'algorithmic_bytes': byt, 'gb_per_s_cold': round(byt / t_cold / 1e9, 1),
                           'frac_of_hbm_peak_cold': round(byt / t_cold / 1e9 / PEAK_HBM_GBPS, 4)}
        del xs, ws
        # fp32 GEMM (fp32 MFMA, 157.3 TFLOP/s peak): a large square, the largest shape of the reference's fp32 test and
        # its m = 128 shape with the fewest outputs, each next to torch.matmul (hipBLASLt) on the same operands
        for mm, nn, kk in ((8192, 8192, 8192), (4096, 7168, 16384), (128, 2112, 7168)):
            a, b, c = harness.make_float_case(mm, nn, kk, seed=42, device='cuda', gen_device='cuda')
            reps = 10 if mm > 128 else 200
            ms, _ = _event_time_ms(lambda: yan.gemm_float_nt(a, b, c), reps, 3)
            ms_t, _ = _event_time_ms(lambda: torch.matmul(a, b.t(), out=c), reps, 3)
            fl = 2.0 * mm * nn * kk
            extra[f'fp32_{mm}x{nn}x{kk}'] = {'us': round(ms * 1e3, 1), 'tflops': round(fl / ms / 1e9, 1),
                                             'frac_of_fp32_peak': round(fl / ms / 1e9 / PEAK_FP32_TFLOPS, 4),
                                             'torch_hipblaslt_us': round(ms_t * 1e3, 1)}
            del a, b, c
    if extra:
        line['extra'] = extra

    if not args.no_cpu:
        line['cpu_baseline'] = _cpu_baseline_fp8(a8, sa, b8, sb)
    else:
        line['cpu_baseline'] = None
    print(json.dumps(line), flush=True)


if __name__ == '__main__':
    main()
