#!/usr/bin/env python3
"""Benchmark of the channels-last 3D depthwise-conv hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--channels 64] [--no-cpu-baseline]

One "step" is one pass of the hot path over one synthetic batch that is already resident in
HBM: DWConv forward followed by DWConvWGRAD at the README shape (1, C, 350, 350, 128), fp16,
channels_last_3d (the README-shape forward and weight-gradient target configurations).  The script prints ONE JSON line:

  metric / value / unit   DWConv fwd + wgrad milliseconds per step (lower is better)
  fwd / wgrad             per-op ms, algorithmic GB/s (4*V*C bytes), % of the 8 TB/s HBM peak and
                          % of the bandwidth torch.clone reaches on the same tensor in this run
  roofline                the dominant kernel of the step, timed live with HIP events on the
                          stream the kernels run on
  ops                     the same figures for every other op of the path (statistics, BN-ReLU, pooling,
                          quantisers, their backward ops, the fused and the linear ops) and for every C of
                          the README table
  cpu_baseline            torch.nn.functional.conv3d(groups=C) in fp32 and its autograd weight gradient on the
                          box's host cores (the CPU baseline the target names; the reference tests' ground
                          truth), at the full shape when the host has the memory for it, else on a crop scaled
                          by the voxel ratio; the CPU oracle (oracle/kerops_oracle.c, OpenMP) is timed beside
                          it on a bounded crop (cpu_oracle_port)

Inputs are synthetic: x, grad ~ N(0, 1) (mean, variance), depthwise weight ~ N(0, 1/27), drawn
with a fixed seed.  Every GPU on this pool is a single-GPU box, so --gpus above 1 is refused.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
H, W, D = 350, 350, 128
V = H * W * D

TRAFFIC_TABLE = os.path.join(ROOT, 'profiles', 'dwconv_hbm_traffic_by_channels.md')
KERNEL_NAMES = {'dwconv_fwd': 'kerops::dwconv_fwd_mfma_kernel', 'dwconv_wgrad': 'kerops::dwconv_wgrad_dma_kernel'}


def load_traffic_table(path=TRAFFIC_TABLE):
    """HBM bytes per launch of the two convolution kernels, per channel count, from the committed rocprofv3 summary
    (rows `| C | kernel | FETCH_SIZE KiB | WRITE_SIZE KiB | HBM bytes | ...`, measured at the commit the file
    names).  Returns ({(kernel, C): bytes}, commit or None); an unreadable file gives an empty table."""
    import re
    table, commit = {}, None
    try:
        text = open(path).read()
    except OSError:
        return table, commit
    m = re.search(r'measured at commit `?([0-9a-f]{7,40})`?', text)
    commit = m.group(1) if m else None
    for row in re.findall(r'^\|\s*(\d+)\s*\|\s*`?(dwconv_\w+)`?\s*\|[^|]*\|[^|]*\|\s*(\d+)\s*\|', text, flags=re.M):
        table[(row[1], int(row[0]))] = int(row[2])
    return table, commit


def clock_under_load(torch, ops, seconds=1.2):
    """Core clock (MHz) that rocm-smi reports while one op runs back to back for `seconds`: the matrix-core
    convolution kernels draw enough power for the clock to come down from its 2.4 GHz ceiling, the pure stream
    kernels do not, and the convolution kernels' time follows the clock.  A reported side figure; None when
    rocm-smi is not there."""
    import re
    import subprocess
    import threading
    out = {}
    for name, fn in ops.items():
        samples, stop = [], threading.Event()

        def sampler():
            while not stop.is_set():
                try:
                    r = subprocess.run(['rocm-smi', '--showclocks', '--json'], capture_output=True, text=True, timeout=5)
                    m = re.search(r'"sclk clock speed:":\s*"\((\d+)Mhz\)"', r.stdout)
                    if m:
                        samples.append(int(m.group(1)))
                except Exception:
                    return
        th = threading.Thread(target=sampler)
        t0 = time.perf_counter()
        n = 0
        th.start()
        while time.perf_counter() - t0 < seconds:
            for _ in range(40):
                fn()
            torch.cuda.synchronize()
            n += 40
        ms = (time.perf_counter() - t0) * 1e3 / n
        stop.set()
        th.join()  # the last rocm-smi call (bounded by its own timeout) returns before the run goes on
        body = samples[1:] if len(samples) > 2 else samples  # the first sample may predate the load
        out[name] = {'sclk_mhz': median(body) if body else None, 'samples': len(samples), 'ms_back_to_back': round(ms, 4)}
    return out


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--channels', type=int, default=64, help='C of the timed step (README table: 8..128)')
    ap.add_argument('--no-cpu-baseline', action='store_true', help='skip the CPU legs (used under rocprofv3)')
    ap.add_argument('--no-extra-ops', action='store_true', help='time only the DWConv step')
    ap.add_argument('--no-clock-probe', action='store_true', help='skip the core-clock-under-load side figure')
    ap.add_argument('--one-shape-per-kernel', action='store_true',
                    help='counter runs: leave out the launches that run a kernel template at a second tensor size '
                         '(stream ops and fused backward at the other channel counts, the C=128 convolution rows), so '
                         'that per-kernel averages of a profiler are averages over one shape')
    return ap.parse_args()


def median(xs):
    s = sorted(xs)
    return s[len(s) // 2]


def time_op(torch, fn, iters, warm):
    """Median / min of per-launch HIP-event times on torch's current stream.  Warm-up: at least `warm` launches and
    at least 30 ms of back-to-back launches, the time the core clock takes to settle after an idle gap (allocations
    and host work between two ops are such gaps; a 0.15 ms kernel would otherwise be timed on the ramp)."""
    t0 = time.perf_counter()
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    while time.perf_counter() - t0 < 0.03:
        for _ in range(max(warm, 5)):
            fn()
        torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    ts = [a.elapsed_time(b) for a, b in evs]
    return median(ts), min(ts), sum(ts) / len(ts)


def figures(ms, nbytes, clone_gbps):
    gbps = nbytes / ms / 1e6
    return {'ms': round(ms, 4), 'GBps': round(gbps, 1), 'frac_hbm_peak': round(gbps / HBM_PEAK_GBPS, 4),
            'frac_of_clone': round(gbps / clone_gbps, 4) if clone_gbps else None, 'algorithmic_bytes': nbytes}


def host_memory_gib():
    """(total, available) host memory in GiB, from /proc/meminfo."""
    info = {}
    try:
        for line in open('/proc/meminfo'):
            k, v = line.split(':', 1)
            info[k] = int(v.split()[0]) / 2 ** 20
    except OSError:
        return None, None
    return info.get('MemTotal'), info.get('MemAvailable')


def cpu_baseline(torch, C, x_dev, g_dev, wk_dev):
    """The host baselines.  Returns (torch conv3d figures, oracle port figures)."""
    import oracle
    from torch.nn import functional as F

    total_gib, avail_gib = host_memory_gib()
    # fp32 x, grad, y and the weight-gradient pass's temporaries: about 16 bytes * 3 per element, with headroom
    need_gib = 3 * 4 * V * C * 4 / 2 ** 30
    full = avail_gib is not None and avail_gib >= need_gib
    hh = H if full else 176
    ww = W if full else 176
    vox = hh * ww * D
    scale = V / vox
    # the same synthetic tensors as the GPU step (leading crop when the host is short of memory)
    x16 = x_dev[:, :, :hh, :ww].contiguous(memory_format=torch.channels_last_3d).cpu()
    g16 = g_dev[:, :, :hh, :ww].contiguous(memory_format=torch.channels_last_3d).cpu()
    wk = wk_dev.cpu()
    wt = wk.permute(3, 0, 1, 2).unsqueeze(1).contiguous()  # (C,1,3,3,3), the layout torch wants

    xf, gf = x16.float(), g16.float()
    w32 = wt.float().requires_grad_(True)
    ts_f, ts_w = [], []
    reps = 3
    for _ in range(reps):
        t0 = time.perf_counter()
        y = F.conv3d(xf, w32, None, 1, 1, 1, C)
        ts_f.append(time.perf_counter() - t0)
        t0 = time.perf_counter()
        (gw,) = torch.autograd.grad(y, w32, gf)
        ts_w.append(time.perf_counter() - t0)
        del y, gw
    del xf, gf
    t_f, t_w = median(ts_f), median(ts_w)
    where = (f'full shape (1,{C},{H},{W},{D})' if full else
             f'leading crop (1,{C},{hh},{ww},{D}), times scaled by the voxel ratio {scale:.2f} '
             f'(host memory available {avail_gib} GiB < {need_gib:.0f} GiB wanted for the full shape)')
    torch_cpu = {
        'value': round((t_f + t_w) * 1e3 * scale, 1), 'unit': 'ms', 'cores': torch.get_num_threads(), 'kind': 'reference',
        'kind_note': 'torch.nn.functional.conv3d(groups=C) on the host, the library routine the reference tests use as '
                     'ground truth (tests/ops/test_conv.py:25,62-72) and the CPU baseline the target names; not a build '
                     'of the reference (which is Python/Triton and has no CPU path)',
        'sample': f'fp32 conv3d(groups={C}) forward + autograd weight gradient, median of {reps} runs, {where}',
        'fwd_ms': round(t_f * 1e3 * scale, 1), 'wgrad_ms': round(t_w * 1e3 * scale, 1),
        'torch_num_threads': torch.get_num_threads(), 'host_cpus': os.cpu_count(),
        'host_memory_gib': {'total': round(total_gib, 1) if total_gib else None,
                            'available': round(avail_gib, 1) if avail_gib else None},
        'full_shape': full,
    }

    # the oracle port on a bounded crop
    crop = (176, 176)
    xo = x16[:, :, :crop[0], :crop[1]].contiguous(memory_format=torch.channels_last_3d)
    go = g16[:, :, :crop[0], :crop[1]].contiguous(memory_format=torch.channels_last_3d)
    oscale = V / (crop[0] * crop[1] * D)
    oracle.dwconv_fwd(xo[:, :, :8], wk, wide=False)  # load the library, warm the thread pool
    reps_f, reps_w = 6, 4
    t0 = time.perf_counter()
    for _ in range(reps_f):
        oracle.dwconv_fwd(xo, wk, wide=False)
    o_f = (time.perf_counter() - t0) / reps_f
    t0 = time.perf_counter()
    for _ in range(reps_w):
        oracle.dwconv_wgrad(xo, go)
    o_w = (time.perf_counter() - t0) / reps_w
    port = {
        'value': round((o_f + o_w) * 1e3 * oscale, 1), 'unit': 'ms', 'cores': oracle.num_threads(), 'kind': 'port',
        'sample': f'oracle DWConv fwd (fp32, {reps_f} runs) + wgrad (fp64, {reps_w} runs) on the leading crop '
                  f'(1,{C},{crop[0]},{crop[1]},{D}), time scaled by the voxel ratio {oscale:.2f} to (1,{C},{H},{W},{D})',
        'fwd_ms_scaled': round(o_f * 1e3 * oscale, 1), 'wgrad_ms_scaled': round(o_w * 1e3 * oscale, 1),
        'host_cpus': os.cpu_count(),
    }
    return torch_cpu, port


def main():
    args = parse()
    if args.gpus != 1:
        print(f'bench.py: every GPU box of this pool has one GPU and the hot path is a single-GPU kernel path; '
              f'--gpus {args.gpus} is not supported (run with --gpus 1)', file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print('bench.py: no ROCm device visible; the benchmark measures HIP kernels only', file=sys.stderr)
        sys.exit(3)
    from kerops_amd.ops.avgpool import AvgPoolCeilStats
    from kerops_amd.ops.bnrelu import ApplyBNReLU
    from kerops_amd.ops.conv import DWConv, DWConvWGRAD
    from kerops_amd.ops.quantization import QuantUint8Window
    from kerops_amd.ops.stats import Stats

    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    C = args.channels
    gen = torch.Generator(dev).manual_seed(322)

    def make(c):
        x = torch.randn(1, H, W, D, c, device=dev, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
        g = torch.randn(1, H, W, D, c, device=dev, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
        wk = (torch.randn(c, 1, 3, 3, 3, device=dev, generator=gen) / math.sqrt(27)).half()
        return x, g, wk[:, 0].permute(1, 2, 3, 0).contiguous()

    x, g, wk = make(C)
    nbytes = 4 * V * C

    # ---- copy floor on the same tensor
    clone_ms, clone_min, _ = time_op(torch, lambda: x.clone(), 30, 5)
    clone_gbps = nbytes / clone_ms / 1e6

    # ---- settle: from idle the GPU takes about 20 steps (30 ms) to reach its steady clocks (per-step times fall
    # from 0.83 to 0.75 ms); run the step untimed for 25 iterations first, so that the figure does not depend on
    # how many warm-up steps the caller asks for
    settle = 25
    for _ in range(settle):
        DWConv(x, wk)
        DWConvWGRAD(x, g)
    torch.cuda.synchronize()

    # ---- the timed region: W warm-up steps, then exactly K steps
    for _ in range(args.warmup):
        DWConv(x, wk)
        DWConvWGRAD(x, g)
    torch.cuda.synchronize()
    K = args.steps
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(K)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(K):
        ev[k][0].record()
        y = DWConv(x, wk)
        ev[k][1].record()
        gw = DWConvWGRAD(x, g)
        ev[k][2].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    fwd_ts = [e[0].elapsed_time(e[1]) for e in ev]
    wg_ts = [e[1].elapsed_time(e[2]) for e in ev]
    ms_per_step = wall_ms / K
    fwd_avg, wg_avg = sum(fwd_ts) / K, sum(wg_ts) / K
    del y, gw

    fwd = figures(median(fwd_ts), nbytes, clone_gbps)
    fwd['ms_avg'], fwd['ms_min'] = round(fwd_avg, 4), round(min(fwd_ts), 4)
    wg = figures(median(wg_ts), nbytes, clone_gbps)
    wg['ms_avg'], wg['ms_min'] = round(wg_avg, 4), round(min(wg_ts), 4)

    traffic_table, traffic_commit = load_traffic_table()
    traffic_note = (f'HBM bytes per launch from profiles/dwconv_hbm_traffic_by_channels.md (rocprofv3 FETCH_SIZE + '
                    f'WRITE_SIZE, measured at commit {traffic_commit})' if traffic_table else
                    'null: profiles/dwconv_hbm_traffic_by_channels.md is missing or holds no row for this channel count')
    dom_name, dom_avg = ('dwconv_wgrad', wg_avg) if wg_avg >= fwd_avg else ('dwconv_fwd', fwd_avg)
    achieved = nbytes / dom_avg / 1e6
    roofline = {
        'kernel': KERNEL_NAMES[dom_name],
        'bound': 'hbm', 'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBPS, 'unit': 'GB/s',
        'frac': round(achieved / HBM_PEAK_GBPS, 4), 'traffic': traffic_table.get((dom_name, C)),
        'traffic_source': traffic_note, 'algorithmic_bytes': nbytes, 'avg_launch_ms': round(dom_avg, 4),
        'note': 'avg over the timed steps of HIP events around the op on the launch stream; for wgrad the '
                'launch includes its partial-sum reduce kernel (~1% of the time)',
    }
    other = 'dwconv_fwd' if dom_name == 'dwconv_wgrad' else 'dwconv_wgrad'
    other_avg = fwd_avg if other == 'dwconv_fwd' else wg_avg
    roofline_other = {
        'kernel': KERNEL_NAMES[other], 'bound': 'hbm', 'achieved': round(nbytes / other_avg / 1e6, 1),
        'peak': HBM_PEAK_GBPS, 'unit': 'GB/s', 'frac': round(nbytes / other_avg / 1e6 / HBM_PEAK_GBPS, 4),
        'traffic': traffic_table.get((other, C)), 'algorithmic_bytes': nbytes,
        'avg_launch_ms': round(other_avg, 4),
    }

    ops = {}
    if not args.no_extra_ops:
        Wv = torch.rand(C, device=dev, generator=gen) + 0.5
        Bv = torch.randn(C, device=dev, generator=gen) * 0.3
        it, wm = 20, 3
        ops['Stats'] = figures(time_op(torch, lambda: Stats(x), it, wm)[0], 2 * V * C, clone_gbps)
        ops['ApplyBNReLU'] = figures(time_op(torch, lambda: ApplyBNReLU(x, Wv, Bv), it, wm)[0], 4 * V * C, clone_gbps)
        ops['AvgPoolCeilStats'] = figures(time_op(torch, lambda: AvgPoolCeilStats(x), it, wm)[0],
                                          2 * V * C + 2 * (V // 8) * C, clone_gbps)
        from kerops_amd.ops.avgpool import ApplyBNReLUAvgPoolCeilStats
        ops['ApplyBNReLU+AvgPoolCeilStats_fused'] = figures(
            time_op(torch, lambda: ApplyBNReLUAvgPoolCeilStats(x, Wv, Bv), it, wm)[0], 2 * V * C * (1 + 1 / 8),
            clone_gbps)
        from kerops_amd.ops.conv import DWConvStats
        ops['DWConv+Stats_fused'] = figures(time_op(torch, lambda: DWConvStats(x, wk), it, wm)[0], 4 * V * C, clone_gbps)
        ops['DWConv+Stats_fused']['note'] = 'replaces DWConv + Stats on its output (fwd.ms + ops.Stats.ms)'
        from kerops_amd.ops.conv import DWConvBackward
        ops['DWConvBackward_fused'] = figures(time_op(torch, lambda: DWConvBackward(x, g, wk), it, wm)[0], 6 * V * C,
                                              clone_gbps)
        ops['QuantUint8Window'] = figures(time_op(torch, lambda: QuantUint8Window(x, 3.0), it, wm)[0], 3 * V * C,
                                          clone_gbps)
        # the remaining stream ops (backward passes, residual add, dequantiser) on the same tensor
        from kerops_amd.ops.addition import AddStats, AddStatsBackward
        from kerops_amd.ops.avgpool import AvgPoolCeilStatsBackward
        from kerops_amd.ops.bnrelu import ApplyBNReLUBackward
        from kerops_amd.ops.quantization import DequantUint8Window
        from kerops_amd.ops.stats import StatsBackward
        mg = torch.randn(C, device=dev, generator=gen)
        sg = torch.randn(C, device=dev, generator=gen)
        ops['StatsBackward'] = figures(time_op(torch, lambda: StatsBackward(x, mg, sg), it, wm)[0], 4 * V * C, clone_gbps)
        ops['AddStats'] = figures(time_op(torch, lambda: AddStats(x, g), it, wm)[0], 6 * V * C, clone_gbps)
        ops['AddStatsBackward'] = figures(time_op(torch, lambda: AddStatsBackward(g, mg, sg, x), it, wm)[0], 6 * V * C,
                                          clone_gbps)
        ops['ApplyBNReLUBackward'] = figures(time_op(torch, lambda: ApplyBNReLUBackward(x, Wv, Bv, g), it, wm)[0],
                                             6 * V * C, clone_gbps)
        pooled = AvgPoolCeilStats(x)[0]
        gp = torch.randn_like(pooled)
        ops['AvgPoolCeilStatsBackward'] = figures(
            time_op(torch, lambda: AvgPoolCeilStatsBackward(gp, mg, sg, pooled, tuple(x.shape)), it, wm)[0],
            2 * V * C + 4 * pooled.numel(), clone_gbps)
        q8 = QuantUint8Window(x, 3.0)
        ops['DequantUint8Window'] = figures(time_op(torch, lambda: DequantUint8Window(q8, torch.float16, 3.0), it, wm)[0],
                                            3 * V * C, clone_gbps)
        del pooled, gp, q8
        # the vendor path on the same GPU: torch's own depthwise conv3d (MIOpen) on the same tensor, forward only
        # (its weight gradient takes 2.5 s per call after a 78 s kernel search, so it is not run here)
        try:
            import torch.nn.functional as F
            wt_t = wk.permute(3, 0, 1, 2).unsqueeze(1).contiguous()
            t_ms = time_op(torch, lambda: F.conv3d(x, wt_t, None, 1, 1, 1, C), 3, 1)[0]
            ops['gpu_torch_conv3d_groups'] = {'fwd_ms': round(t_ms, 2), 'vs_DWConv': round(t_ms / fwd['ms'], 1),
                                              'note': 'torch.nn.functional.conv3d(groups=C), fp16 channels_last_3d, '
                                                      'same tensor, same GPU; median of 3 after 1 warm-up'}
            del wt_t
        except Exception as e:  # a reported side figure only
            ops['gpu_torch_conv3d_groups'] = {'error': repr(e)[:200]}
        def stream_rows(xc, gc, c):
            """Every stream op at (1,c,350,350,128): ms and fraction of the HBM peak of its algorithmic bytes."""
            wv = torch.rand(c, device=dev, generator=gen) + 0.5
            bv = torch.randn(c, device=dev, generator=gen) * 0.3
            mgc = torch.randn(c, device=dev, generator=gen)
            sgc = torch.randn(c, device=dev, generator=gen)
            pooled_c = AvgPoolCeilStats(xc)[0]
            gpc = torch.randn_like(pooled_c)
            q8c = QuantUint8Window(xc, 3.0)
            amax = torch.full((1,), 5.0, device=dev)
            vc = V * c
            cases = [
                ('Stats', lambda: Stats(xc), 2 * vc), ('StatsBackward', lambda: StatsBackward(xc, mgc, sgc), 4 * vc),
                ('AddStats', lambda: AddStats(xc, gc), 6 * vc),
                ('AddStatsBackward', lambda: AddStatsBackward(gc, mgc, sgc, xc), 6 * vc),
                ('ApplyBNReLU', lambda: ApplyBNReLU(xc, wv, bv), 4 * vc),
                ('ApplyBNReLUBackward', lambda: ApplyBNReLUBackward(xc, wv, bv, gc), 6 * vc),
                ('AvgPoolCeilStats', lambda: AvgPoolCeilStats(xc), 2 * vc + 2 * pooled_c.numel()),
                ('ApplyBNReLU+AvgPoolCeilStats_fused', lambda: ApplyBNReLUAvgPoolCeilStats(xc, wv, bv),
                 2 * vc + 2 * pooled_c.numel()),
                ('AvgPoolCeilStatsBackward', lambda: AvgPoolCeilStatsBackward(gpc, mgc, sgc, pooled_c, tuple(xc.shape)),
                 2 * vc + 4 * pooled_c.numel()),
                ('QuantUint8Window', lambda: QuantUint8Window(xc, 3.0), 3 * vc),
                ('DequantUint8Window', lambda: DequantUint8Window(q8c, torch.float16, 3.0), 3 * vc),
                ('QuantInt8Sym', lambda: QuantInt8Sym(xc, amax), 3 * vc),
            ]
            if args.one_shape_per_kernel:
                cases = cases[:-1]  # (QuantInt8Sym runs at the config-5 shape below)
            rows = {}
            for name, fn, nb in cases:
                ms_ = time_op(torch, fn, it, wm)[0]
                rows[name] = {'ms': round(ms_, 4), 'frac_hbm_peak': round(nb / ms_ / 1e6 / HBM_PEAK_GBPS, 4)}
            return rows

        from kerops_amd.ops.quantization import QuantInt8Sym
        table, stream_table = {}, {str(C): stream_rows(x, g, C)}  # (x, g still hold the C-channel tensors here)
        for c in (8, 16, 32, 64, 128):
            if c == C:
                table[str(c)] = {'clone_ms': round(clone_ms, 4), 'dwconv_ms': fwd['ms'], 'wgrad_ms': wg['ms'],
                                 'dwconv_frac_of_clone': fwd['frac_of_clone'],
                                 'wgrad_frac_of_clone': wg['frac_of_clone'],
                                 'dwconv_frac_hbm_peak': fwd['frac_hbm_peak'],
                                 'wgrad_frac_hbm_peak': wg['frac_hbm_peak']}
                continue
            if args.one_shape_per_kernel and c in (64, 128):  # (these two share their kernel templates)
                continue
            x = g = None
            torch.cuda.empty_cache()
            x, g, wkc = make(c)
            cm = time_op(torch, lambda: x.clone(), it, wm)[0]
            fm = time_op(torch, lambda: DWConv(x, wkc), it, wm)[0]
            wgm = time_op(torch, lambda: DWConvWGRAD(x, g), it, wm)[0]
            bwm = time_op(torch, lambda: DWConvBackward(x, g, wkc), it, wm)[0]
            table[str(c)] = {'clone_ms': round(cm, 4), 'dwconv_ms': round(fm, 4), 'wgrad_ms': round(wgm, 4),
                             'dwconv_frac_of_clone': round(cm / fm, 4), 'wgrad_frac_of_clone': round(cm / wgm, 4),
                             'dwconv_frac_hbm_peak': round(4 * V * c / fm / 1e6 / HBM_PEAK_GBPS, 4),
                             'wgrad_frac_hbm_peak': round(4 * V * c / wgm / 1e6 / HBM_PEAK_GBPS, 4),
                             'backward_fused_ms': round(bwm, 4),
                             'backward_fused_frac_hbm_peak': round(6 * V * c / bwm / 1e6 / HBM_PEAK_GBPS, 4)}
            if not args.one_shape_per_kernel:
                stream_table[str(c)] = stream_rows(x, g, c)
        table[str(C)]['backward_fused_ms'] = ops['DWConvBackward_fused']['ms']
        table[str(C)]['backward_fused_frac_hbm_peak'] = ops['DWConvBackward_fused']['frac_hbm_peak']
        ops['stream_ops_by_channels'] = {str(c): stream_table[str(c)] for c in (8, 16, 32, 64, 128) if str(c) in stream_table}
        ops['stream_ops_by_channels_note'] = ('every stream op at (1,C,350,350,128) with the launch shape of the table '
                                              'entry for that C (kerops_amd/settings/stream_shapes.json)')
        ops['readme_table'] = table
        # target configuration 5: fused depthwise-separable block with int8 output at (1,64,128,128,128)
        del x, g
        torch.cuda.empty_cache()
        from kerops_amd.ops.fused import DWSepBlock, PointwiseLinear
        from kerops_amd.ops.quantization import QuantInt8Sym
        V5 = 128 ** 3
        x5 = torch.randn(1, 128, 128, 128, 64, device=dev, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
        wk5 = (torch.randn(3, 3, 3, 64, device=dev, generator=gen) / math.sqrt(27)).half()
        sc5 = torch.rand(64, device=dev, generator=gen) + 0.5
        sh5 = torch.randn(64, device=dev, generator=gen) * math.sqrt(0.1)
        Wm5 = (torch.randn(64, 128, device=dev, generator=gen) / 8.0).half()
        stage1_bytes = 2 * V5 * 64 + 2 * V5 * 128
        c5 = time_op(torch, lambda: x5.clone(), it, wm)[0]
        c5_gbps = 4 * V5 * 64 / c5 / 1e6
        ops['config5_block_stage1'] = figures(time_op(torch, lambda: DWSepBlock(x5, wk5, sc5, sh5, Wm5), it, wm)[0],
                                              stage1_bytes, c5_gbps)
        ops['config5_pointwise_64_128'] = figures(time_op(torch, lambda: PointwiseLinear(x5, Wm5), it, wm)[0],
                                                  stage1_bytes, c5_gbps)
        y5, am5 = DWSepBlock(x5, wk5, sc5, sh5, Wm5)
        ops['config5_int8_pass'] = figures(time_op(torch, lambda: QuantInt8Sym(y5, am5), it, wm)[0], 3 * V5 * 128,
                                           c5_gbps)
        # pointwise ops of the reference's linear family at (1,32,350,350,128) (its tests use 32 channels)
        from kerops_amd.ops.linear import LinBReLULinAdd, LinBReLULinBackward, ReLULinearAdd, ReLULinearBackward
        del y5
        cl = 32
        xl = torch.randn(1, 350, 350, 128, cl, device=dev, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
        gl = torch.randn(1, 350, 350, 128, cl, device=dev, dtype=torch.float16, generator=gen).permute(0, 4, 1, 2, 3)
        Wl = (torch.randn(cl, cl, device=dev, generator=gen) / math.sqrt(cl)).half()
        Wu = (torch.randn(cl, 2 * cl, device=dev, generator=gen) / math.sqrt(cl)).half()
        Wd = (torch.randn(2 * cl, cl, device=dev, generator=gen) / math.sqrt(2 * cl)).half()
        bl = (torch.randn(2 * cl, device=dev, generator=gen) * 0.5).half()
        cl_ms = time_op(torch, lambda: xl.clone(), it, wm)[0]
        cl_gbps = 4 * V * cl / cl_ms / 1e6
        ops['ReLULinearAdd_32_32'] = figures(time_op(torch, lambda: ReLULinearAdd(xl, Wl, gl), it, wm)[0],
                                             6 * V * cl, cl_gbps)
        from kerops_amd.ops.linear import ApplyBNReLULinearAdd
        bwl = torch.rand(cl, device=dev, generator=gen) + 0.5
        bbl = torch.randn(cl, device=dev, generator=gen) * 0.3
        ops['ApplyBNReLU+ReLULinearAdd_fused_32_32'] = figures(
            time_op(torch, lambda: ApplyBNReLULinearAdd(xl, bwl, bbl, Wl, gl), it, wm)[0], 6 * V * cl, cl_gbps)
        ops['ApplyBNReLU+ReLULinearAdd_fused_32_32']['note'] = (
            'replaces ApplyBNReLU (4*V*C bytes more) + ReLULinearAdd, bit-identical')
        ops['ReLULinearBackward_32_32'] = figures(time_op(torch, lambda: ReLULinearBackward(xl, gl, Wl), it, wm)[0],
                                                  6 * V * cl, cl_gbps)
        ops['LinBReLULinAdd_32'] = figures(time_op(torch, lambda: LinBReLULinAdd(xl, Wu, Wd, bl, gl), it, wm)[0],
                                           6 * V * cl, cl_gbps)
        ops['LinBReLULinBackward_32'] = figures(
            time_op(torch, lambda: LinBReLULinBackward(xl, gl, Wu, Wd, bl), it, wm)[0], 6 * V * cl, cl_gbps)
        del xl, gl
        ops['config5_note'] = ('stage 1 = one kernel: matrix-core DWConv, BN+ReLU, fp16 tile through LDS into the MFMA '
                               '1x1x1 GEMM with fused max|y|; the 64-channel intermediate never reaches memory')
        ops['readme_table_note'] = 'C=8 (251 MB) fits the 256 MB Infinity Cache: its rows are not pure HBM numbers'

    clocks = None
    if not args.no_clock_probe:
        xs, gs, wks = make(C)
        from kerops_amd.ops.bnrelu import ApplyBNReLU as _bn
        ones, zeros = torch.ones(C, device=dev), torch.zeros(C, device=dev)
        probes = {'DWConv': lambda: DWConv(xs, wks), 'DWConvWGRAD': lambda: DWConvWGRAD(xs, gs),
                  'ApplyBNReLU': lambda: _bn(xs, ones, zeros)}
        if not args.no_extra_ops:
            from kerops_amd.ops.conv import DWConvBackward as _bwd, DWConvStats as _cs
            from kerops_amd.ops.fused import DWSepBlock as _blk, PointwiseLinear as _pw
            probes['DWConvStats'] = lambda: _cs(xs, wks)
            probes['DWConvBackward'] = lambda: _bwd(xs, gs, wks)
            if C == 64:
                Wp = (torch.randn(64, 128, device=dev, generator=gen) / 8.0).half()
                probes['DWSepBlock_64_128'] = lambda: _blk(xs, wks, ones, zeros, Wp)
                probes['PointwiseLinear_64_128'] = lambda: _pw(xs, Wp)
        clocks = clock_under_load(torch, probes)
        clocks['note'] = ('rocm-smi sclk sampled while the op runs back to back on the (1,C,350,350,128) tensor; '
                          'ceiling 2400 MHz')
        del xs, gs

    cpu, cpu_port = (None, None)
    if not args.no_cpu_baseline:
        xs, gs, wks = make(C)
        cpu, cpu_port = cpu_baseline(torch, C, xs, gs, wks)
        del xs, gs

    out = {
        'metric': f'DWConv fwd/wgrad ms + % HBM roofline, fp16 (1,{C},350,350,128) NDHWC',
        'value': round(ms_per_step, 4), 'unit': 'ms', 'n_gpus': 1, 'steps': K, 'warmup': args.warmup,
        'ms_per_step': round(ms_per_step, 4), 'higher_is_better': False, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'f16 in/out, f32 accumulate', 'data': 'synthetic',
        'config': {'workload': f'DWConv fwd + DWConvWGRAD, x/grad fp16 channels_last_3d (1,{C},350,350,128), '
                               'weight [3,3,3,C], pad 1, stride 1 (target configurations 2 and 3)',
                   'channels': C, 'voxels': V, 'inputs_resident_in_hbm': True},
        'settle_steps_before_warmup': settle,
        'fwd': fwd, 'wgrad': wg,
        'clone': {'ms': round(clone_ms, 4), 'ms_min': round(clone_min, 4), 'GBps': round(clone_gbps, 1),
                  'frac_hbm_peak': round(clone_gbps / HBM_PEAK_GBPS, 4)},
        'targets': {'fwd_frac_of_clone>=0.75': fwd['frac_of_clone'] >= 0.75,
                    'wgrad_frac_of_clone>=0.50': wg['frac_of_clone'] >= 0.50},
        'roofline': roofline, 'roofline_other': roofline_other,
        'core_clock_under_load': clocks,
        'cpu_baseline': cpu, 'cpu_oracle_port': cpu_port, 'ops': ops,
        'device': torch.cuda.get_device_name(0),
    }
    print(json.dumps(out))


if __name__ == '__main__':
    main()
