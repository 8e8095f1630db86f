"""Measure the built launch shapes of the ops on the GPU at hand and install the winners.

The reference ships static per-channel tables tuned for one card (kerops/ops/conv/dwconv.py:10-17,
kerops/ops/conv/dwconv_wgrad.py:10-22); the tables in kerops_amd/ops/conv were measured on an MI355X at
(1, C, 350, 350, 128).  For another shape or part:

    python -m kerops_amd.tune --shape 1 64 350 350 128          # print the timings
    python -m kerops_amd.tune --channels 32 64 --apply          # and reconfigure the ops of this process

    python -m kerops_amd.tune --streams                         # the flat stream ops: (blocks, num_warps, segment)
    python -m kerops_amd.tune --streams --all --write           # every channel count of the README table and the
                                                                # small-tensor class; rewrites settings/stream_shapes.json

`tune(...)` returns {op: {C: (W_block, D_block, lane_channels, H_chunk, ms)}}; `apply(result)` installs the
choices through the ops' `reconfigure`, the same mechanism a user of the reference has for overriding its tables.
`tune_streams(...)` returns {op: (blocks, num_warps, segment, ms)}; `apply_streams(result, key)` puts them into the
live table of `kerops_amd.settings.stream_table` under a key (a channel count, "small" or "default"), which the
stream ops read on every call.
"""
import argparse
import time
import math

import torch

from .ops.conv import DWConv, DWConvWGRAD
from .ops.conv.variants import FWD_VARIANTS, WGRAD_VARIANTS, threads_per_workgroup


def _time(fn, iters, warmup):
    # at least `warmup` launches and 30 ms of back-to-back launches: the core clock needs that long to settle after an
    # idle gap, and a 0.1 ms kernel timed on the ramp loses to one timed after it
    t0 = time.perf_counter()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    while time.perf_counter() - t0 < 0.03:
        for _ in range(max(warmup, 5)):
            fn()
        torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in evs)
    return ts[len(ts) // 2]


def tune(shape=(1, 64, 350, 350, 128), channels=None, h_chunks=(0,), iters=10, warmup=3, device='cuda', verbose=False):
    """Times every built launch shape for the given (N, C, H, W, D) (C replaced by each entry of `channels`)."""
    n, c0, h, w, d = shape
    result = {'DWConv': {}, 'DWConvWGRAD': {}}
    for c in (channels or [c0]):
        x = torch.randn(n, h, w, d, c, device=device, dtype=torch.float16).permute(0, 4, 1, 2, 3)
        g = torch.randn(n, h, w, d, c, device=device, dtype=torch.float16).permute(0, 4, 1, 2, 3)
        wk = (torch.randn(3, 3, 3, c, device=device) / math.sqrt(27)).half()
        for name, table, run in (
            ('DWConv', FWD_VARIANTS, lambda kw: DWConv(x, wk, **kw)),
            ('DWConvWGRAD', WGRAD_VARIANTS, lambda kw: DWConvWGRAD(x, g, **kw)),
        ):
            best = None
            for (tw, td, cl) in table[c]:
                for hc in h_chunks:
                    kw = dict(W_block=tw, D_block=td, lane_channels=cl, H_chunk=hc,
                              num_warps=threads_per_workgroup(c, tw, td, cl) // 64)
                    ms = _time(lambda: run(kw), iters, warmup)
                    if verbose:
                        print(f'{name:12s} C={c:3d} patch {tw}x{td} lane_channels {cl:2d} H_chunk {hc:3d}: {ms:.3f} ms',
                              flush=True)
                    if best is None or ms < best[4]:
                        best = (tw, td, cl, hc, ms)
            result[name][c] = best
        del x, g
    return result


def _picker(table, idx, fallback):
    def pick(x):
        c = x.shape[1]
        return table[c][idx] if c in table else fallback(c)

    return pick


def _warps_picker(table, fallback):
    def pick(x):
        c = x.shape[1]
        return threads_per_workgroup(c, *table[c][:3]) // 64 if c in table else fallback(c)

    return pick


def apply(result):
    """Installs the measured winners as the ops' defaults (channel counts not measured keep the built-in table)."""
    from .ops.conv import dwconv as fwd_mod, dwconv_wgrad as wg_mod
    for op, mod, key in ((DWConv, fwd_mod, 'DWConv'), (DWConvWGRAD, wg_mod, 'DWConvWGRAD')):
        table = result.get(key, {})
        if not table:
            continue
        conf = dict(op.configurators)
        conf['W_block'] = _picker(table, 0, mod.wtile)
        conf['D_block'] = _picker(table, 1, mod.dblock)
        conf['lane_channels'] = _picker(table, 2, getattr(mod, 'lanec', lambda c: 16))
        conf['H_chunk'] = _picker(table, 3, lambda c: 0)
        conf['num_warps'] = _warps_picker(table, mod.warps)
        op.reconfigure(**conf)


STREAM_BLOCKS = (256, 512, 768, 1024, 1280, 1536, 2048, 3072, 4096)
STREAM_SHAPES = ((4, 1), (4, 4), (4, 8), (16, 1), (16, 4), (16, 8))  # (num_warps, segment)
POOL_SHAPES = ((4, 1), (4, 2), (16, 1), (16, 2))


def stream_cases(shape, device='cuda'):
    """{op name: callable(**knobs)} on synthetic tensors of the given (N, C, H, W, D)."""
    from .ops.addition import AddStats, AddStatsBackward
    from .ops.avgpool import ApplyBNReLUAvgPoolCeilStats, AvgPoolCeilStats, AvgPoolCeilStatsBackward
    from .ops.bnrelu import ApplyBNReLU, ApplyBNReLUBackward
    from .ops.quantization import DequantUint8Window, QuantInt8Sym, QuantUint8Window
    from .ops.stats import Stats, StatsBackward

    n, c, h, w, d = shape
    x = torch.randn(n, h, w, d, c, device=device, dtype=torch.float16).permute(0, 4, 1, 2, 3)
    y = torch.randn(n, h, w, d, c, device=device, dtype=torch.float16).permute(0, 4, 1, 2, 3)
    z = torch.empty_like(x)
    wv = torch.rand(c, device=device) + 0.5
    bv = torch.randn(c, device=device)
    q = torch.randint(0, 256, x.shape, device=device, dtype=torch.uint8).permute(0, 2, 3, 4, 1).contiguous().permute(0, 4, 1, 2, 3)
    amax = torch.full((1,), 5.0, device=device)
    del z
    pooled = AvgPoolCeilStats(x)[0]
    pooled_grad = torch.randn_like(pooled)
    return {
        'AvgPoolCeilStats': lambda **kw: AvgPoolCeilStats(x, **kw),
        'ApplyBNReLUAvgPoolCeilStats': lambda **kw: ApplyBNReLUAvgPoolCeilStats(x, wv, bv, **kw),
        'AvgPoolCeilStatsBackward': lambda **kw: AvgPoolCeilStatsBackward(pooled_grad, wv, bv, pooled, list(x.shape), **kw),
        'Stats': lambda **kw: Stats(x, **kw),
        'StatsBackward': lambda **kw: StatsBackward(x, wv, bv, **kw),
        'AddStats': lambda **kw: AddStats(x, y, **kw),
        'AddStatsBackward': lambda **kw: AddStatsBackward(x, wv, bv, y, **kw),
        'ApplyBNReLU': lambda **kw: ApplyBNReLU(x, wv, bv, **kw),
        'ApplyBNReLUBackward': lambda **kw: ApplyBNReLUBackward(x, wv, bv, y, **kw),
        'QuantUint8Window': lambda **kw: QuantUint8Window(x, 3.0, **kw),
        'DequantUint8Window': lambda **kw: DequantUint8Window(q, torch.float16, 3.0, **kw),
        'QuantInt8Sym': lambda **kw: QuantInt8Sym(x, amax, **kw),
    }


def tune_streams(shape=(1, 64, 350, 350, 128), ops=None, iters=12, warmup=3, rounds=3, device='cuda', verbose=False):
    """Times every (blocks, num_warps, segment) of the built stream kernels; returns {op: (blocks, warps, segment, ms)}.
    Every shape is measured in `rounds` separate passes over the whole table (median of `iters` launches each) and
    scored by the worst of its passes, so that one lucky pass does not pick the shape."""
    result = {}
    for name, run in stream_cases(shape, device).items():
        if ops and name not in ops:
            continue
        table = [(blocks, warps, segment) for warps, segment in (POOL_SHAPES if 'AvgPool' in name else STREAM_SHAPES)
                 for blocks in STREAM_BLOCKS]
        score = {}
        for _ in range(rounds):
            for blocks, warps, segment in table:
                kw = dict(blocks=blocks, num_warps=warps, segment=segment)
                ms = _time(lambda: run(**kw), iters, warmup)
                score[(blocks, warps, segment)] = max(ms, score.get((blocks, warps, segment), 0.0))
        if verbose:
            for (blocks, warps, segment), ms in score.items():
                print(f'{name:20s} blocks {blocks:5d} num_warps {warps:2d} segment {segment}: {ms:.4f} ms', flush=True)
        key = min(score, key=score.get)
        result[name] = key + (score[key],)
    return result


def apply_streams(result, write=False, note='', key='default'):
    from .settings import stream_table
    for op, (blocks, warps, segment, _) in result.items():
        stream_table.set_stream_shape(op, blocks=blocks, num_warps=warps, segment=segment, key=key)
    if write:
        stream_table.save(note=note)


# `--streams --all`: the tensors behind each key of the stream table.  "default" (channel counts without an entry)
# repeats the 64-channel measurement.
STREAM_CLASSES = (('8', (1, 8, 350, 350, 128)), ('16', (1, 16, 350, 350, 128)), ('32', (1, 32, 350, 350, 128)),
                  ('64', (1, 64, 350, 350, 128)), ('128', (1, 128, 350, 350, 128)), ('small', (2, 16, 64, 64, 64)))


def main():
    ap = argparse.ArgumentParser(description=__doc__.split('\n')[0])
    ap.add_argument('--streams', action='store_true', help='tune the flat stream ops instead of the convolution pair')
    ap.add_argument('--write', action='store_true', help='with --streams: rewrite settings/stream_shapes.json')
    ap.add_argument('--ops', nargs='*', default=None, help='with --streams: only these ops')
    ap.add_argument('--all', action='store_true', help='with --streams: every class of the stream table')
    ap.add_argument('--key', default=None, help='with --streams: table key to file the result under (default: the '
                                                'channel count of --shape)')
    ap.add_argument('--shape', type=int, nargs=5, default=[1, 64, 350, 350, 128], metavar=('N', 'C', 'H', 'W', 'D'))
    ap.add_argument('--channels', type=int, nargs='*', default=None)
    ap.add_argument('--h-chunks', type=int, nargs='*', default=[0])
    ap.add_argument('--apply', action='store_true')
    args = ap.parse_args()
    if args.streams:
        classes = STREAM_CLASSES if args.all else ((args.key or str(args.shape[1]), tuple(args.shape)),)
        for key, shape in classes:
            res = tune_streams(shape, ops=args.ops, verbose=not args.all)
            for op, (blocks, warps, segment, ms) in res.items():
                print(f'best {key:>7s} {op:28s}: blocks={blocks} num_warps={warps} segment={segment}  {ms:.4f} ms',
                      flush=True)
            apply_streams(res, key=key)
            if key == '64':
                apply_streams(res, key='default')
        if args.write:
            from .settings import stream_table
            stream_table.save(note='measured by kerops_amd.tune --streams on ' + torch.cuda.get_device_name(0) + ': keys '
                              + ', '.join(f'{k} at {sh}' for k, sh in classes) + '; "default" repeats 64')
        return
    res = tune(tuple(args.shape), args.channels, tuple(args.h_chunks), verbose=True)
    for op, table in res.items():
        for c, (tw, td, cl, hc, ms) in table.items():
            print(f'best {op:12s} C={c:3d}: W_block={tw} D_block={td} lane_channels={cl} H_chunk={hc}  {ms:.3f} ms')
    if args.apply:
        apply(res)


if __name__ == '__main__':
    main()
