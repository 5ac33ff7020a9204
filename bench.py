#!/usr/bin/env python3
"""Benchmark of the dropless-MoE layer hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c3] [--no-cpu]

A step is one forward+backward of the dMoE layer on a batch of synthetic tokens that is
already resident in HBM.  Prints ONE JSON line: whole-job tokens/s, the grouped-GEMM roofline
(algorithmic FLOPs / live HIP-event kernel time vs the bf16 dense MFMA peak), per-kernel
figures for the permutation kernels (algorithmic bytes / kernel time vs the HBM peak), and the
CPU formulation of the same path timed on this host's cores as a baseline.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_PEAK = {'bf16': 2.5e15, 'f16': 2.5e15, 'f32': 157.3e12}
HBM_PEAK = 8e12
# HBM bytes per launch of the grouped-GEMM kernels as rocprofv3 counted them (FETCH_SIZE scaled by what a plain copy of
# known size shows, plus WRITE_SIZE): read from the machine-readable companion of the counter summaries under
# profiles/, so the figure printed is the one of the committed profile and names it.
TRAFFIC_FILE = os.path.join(ROOT, 'profiles', 'hbm_traffic.json')


def measured_traffic(workload, kernel):
    """(bytes per launch or None, where it comes from / why there is none)."""
    try:
        table = json.load(open(TRAFFIC_FILE))
    except (OSError, ValueError) as exc:
        return None, f'{os.path.relpath(TRAFFIC_FILE, ROOT)} unreadable: {exc}'
    entry = table.get('workloads', {}).get(workload, {}).get(kernel)
    if entry is None:
        return None, f'no counter run of {kernel} on {workload} in {os.path.relpath(TRAFFIC_FILE, ROOT)}'
    return entry['bytes_per_launch'], entry.get('source')


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--config', default='c3', choices=['c1', 'c2', 'c3', 'c4', 'c5'])
    ap.add_argument('--tokens', type=int, default=None, help='override the token count (not the headline number)')
    ap.add_argument('--memory-optimized', action='store_true')
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline')
    ap.add_argument('--graph', action='store_true',
                    help='capture the step (forward + backward) in a HIP graph after the warm-up and time replays of it')
    ap.add_argument('--forward-only', action='store_true',
                    help='time the forward pass alone, without gradients (not the headline metric; no CPU baseline)')
    ap.add_argument('--cpu-tokens', type=int, default=None)
    ap.add_argument('--library-gemm', action='store_true',
                    help='also time the three grouped products as per-expert torch.matmul loops (the vendor GEMM library)')
    ap.add_argument('--operand-patterns', action='store_true',
                    help='also time the grouped GEMM launches on all-zero and all-one operands (same shapes): what the '
                         'same instruction stream gives when the operands cost no switching power')
    ap.add_argument('--tile-ticks', action='store_true',
                    help='only: per-tile phase times of the grouped products, from the build with time stamps (libmbx_ticks.so)')
    ap.add_argument('--mfma-ceiling', action='store_true',
                    help='also run a loop of matrix-core instructions alone (no LDS, no memory) on all-zero, all-one and '
                         'N(0,1) bf16 operands: the rate and shader clock the power limit allows on such values')
    ap.add_argument('--calibrate-copy', action='store_true',
                    help='also launch one plain 1 GiB device copy (a known-size reference for HBM byte counters)')
    return ap.parse_args()


def dtype_name(dt):
    import torch
    return {torch.bfloat16: 'bf16', torch.float16: 'f16', torch.float32: 'f32'}[dt]


def gpu_leg(args, w, inp):
    import torch

    from megablocks_amd import _lib, synthetic

    dev = torch.device('cuda', 0)
    torch.cuda.set_device(dev)
    layer = synthetic.build_layer(w, inp, device=dev, memory_optimized=args.memory_optimized)
    x = inp['x'].to(w.dtype).to(dev).requires_grad_(True)
    grad = inp['grad'].to(w.dtype).to(dev)
    routing = None
    if w.routing != 'router':
        ew = inp['expert_weights'].to(w.dtype).to(dev).requires_grad_(True)
        routing = (inp['scores'].to(w.dtype).to(dev), ew, inp['top_experts'].to(dev))

    def step():
        x.grad = None
        if routing is not None:
            routing[1].grad = None
        for p in layer.parameters():
            p.grad = None
        synthetic.layer_step(layer, w, x, grad, routing)

    if args.forward_only:
        if args.graph:
            sys.exit('bench.py: --graph captures the training step; not with --forward-only')

        def step():
            with torch.no_grad():
                return layer(x) if routing is None else layer.experts(x, *routing)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    timed_step = step
    if args.graph:
        if w.mlp_impl == 'sparse':
            sys.exit('bench.py: --graph needs a step without host synchronisation; the block-sparse mode reads the '
                     'padded row count on the host (as the reference does, kernels.py:123-124)')
        step()                      # leaves the gradients unset: the captured step allocates them in the graph's pool
        x.grad = None
        if routing is not None:
            routing[1].grad = None
        for p in layer.parameters():
            p.grad = None
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            synthetic.layer_step(layer, w, x, grad, routing)
        timed_step = graph.replay
        for _ in range(3):
            timed_step()
        torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        timed_step()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = e0.elapsed_time(e1) / args.steps
    ms_wall = wall * 1e3 / args.steps

    # second pass with HIP events around every grouped-GEMM / permutation launch
    _lib.profile_hook = []
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    records, _lib.profile_hook = _lib.profile_hook, None
    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    agg = {}
    for name, meta, a, b in records:
        d = agg.setdefault(name, dict(ms=[], meta=meta))
        d['ms'].append(a.elapsed_time(b))
    return ms_per_step, ms_wall, agg, layer


def summarize(w, agg, slots_scale):
    """Per-kernel algorithmic work / measured time.  `slots_scale` = real slots / rows handed to the
    kernels (< 1 only in block-sparse mode, whose groups are padded to 128 rows)."""
    dn = dtype_name(w.dtype)
    gemm, perm = {}, {}
    for name, d in agg.items():
        m = d['meta']
        avg_ms = statistics.fmean(d['ms'])
        launches = len(d['ms'])
        if name.startswith('gmm'):
            flops = 2.0 * m['rows'] * slots_scale * m['k'] * m['n']
            # algorithmic bytes of the launch: every operand and the output once
            pairs = 2 if name.endswith('_dual') else 1
            kk = m['k'] / pairs
            nbytes = (pairs * (m['rows'] * slots_scale * kk + m['groups'] * kk * m['n']) + m['rows'] * slots_scale * m['n']) \
                * m['elem'] if not name.startswith('gmm_tn') else \
                (m['rows'] * slots_scale * (m['k'] + m['n']) + m['groups'] * m['k'] * m['n']) * m['elem']
            # [rows, n] tensors the epilogues read or write besides the product: its activation; the saved product; the
            # gated activation (half as wide as the two products side by side); x1, x2 and a second gradient
            # ... ; the combined output next to the product (one row per product row: one expert per token)
            for suffix, more in (('_act', 1.0), ('_dact', 1.0), ('_glu', 0.5), ('_dglu', 3.0), ('_scatter', 1.0)):
                if name.endswith(suffix):
                    nbytes += more * m['rows'] * slots_scale * m['n'] * m['elem']
            gemm[name] = dict(avg_ms=round(avg_ms, 4), launches=launches, flops_per_launch=flops,
                              tflops=round(flops / (avg_ms * 1e-3) / 1e12, 1),
                              frac_of_mfma_peak=round(flops / (avg_ms * 1e-3) / MFMA_PEAK[dn], 4),
                              bytes_per_launch=nbytes, gbps=round(nbytes / (avg_ms * 1e-3) / 1e9, 1),
                              frac_of_hbm_peak=round(nbytes / (avg_ms * 1e-3) / HBM_PEAK, 4))
        elif 'hidden' in m:
            # scatter_backward (weighted gather and router-weight gradient in one pass) also reads the routed rows
            rows_moved = w.tokens + (2 if name == 'scatter_backward' else 1) * w.slots
            nbytes = float(rows_moved) * m['hidden'] * m['elem']
            perm[name] = dict(avg_ms=round(avg_ms, 4), launches=launches, bytes_per_launch=nbytes,
                              gbps=round(nbytes / (avg_ms * 1e-3) / 1e9, 1),
                              frac_of_hbm_peak=round(nbytes / (avg_ms * 1e-3) / HBM_PEAK, 4))
    return gemm, perm


def library_gemm_leg(w, inp):
    """The grouped products of one layer step done the way a build without a grouped kernel does them: one
    library GEMM (torch.matmul, i.e. hipBLASLt / rocBLAS) per expert, on this workload's shapes and its own
    rows-per-expert.  A reference point for the grouped kernel, not part of the layer that is benchmarked."""
    import torch

    dev = torch.device('cuda', 0)
    if w.routing == 'router':
        logits = inp['x'].to(dev).float() @ inp['router_weight'].to(dev).float().t()
        top = logits.topk(w.top_k, dim=-1).indices
    else:
        top = inp['top_experts'].to(dev)
    counts = torch.bincount(top.flatten(), minlength=w.experts).tolist()
    rows = sum(counts)
    a = torch.randn(rows, w.hidden, device=dev, dtype=w.dtype)
    mid = torch.randn(rows, w.ffn, device=dev, dtype=w.dtype)
    w1 = torch.randn(w.experts, w.ffn, w.hidden, device=dev, dtype=w.dtype) * 0.02
    out_f = torch.empty(rows, w.ffn, device=dev, dtype=w.dtype)
    out_h = torch.empty(rows, w.hidden, device=dev, dtype=w.dtype)
    dw = torch.empty(w.experts, w.ffn, w.hidden, device=dev, dtype=w.dtype)
    bounds, start = [], 0
    for c in counts:
        bounds.append((start, start + c))
        start += c

    def nt():   # x @ w1[e]^T
        for e, (lo, hi) in enumerate(bounds):
            if hi > lo:
                torch.matmul(a[lo:hi], w1[e].t(), out=out_f[lo:hi])

    def nn():   # h @ w2[e] (w2 stored like w1: [ffn, hidden])
        for e, (lo, hi) in enumerate(bounds):
            if hi > lo:
                torch.matmul(mid[lo:hi], w1[e], out=out_h[lo:hi])

    def tn():   # h^T @ dy: the weight gradient
        for e, (lo, hi) in enumerate(bounds):
            if hi > lo:
                torch.matmul(mid[lo:hi].t(), a[lo:hi], out=dw[e])
            else:
                dw[e].zero_()

    flops = 2.0 * rows * w.hidden * w.ffn
    res = {'what': 'one torch.matmul per expert (vendor GEMM library), same shapes and rows per expert', 'kernels': {}}
    for name, fn in (('gmm_nt', nt), ('gmm_nn', nn), ('gmm_tn', tn)):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / 10
        res['kernels'][name] = dict(avg_ms=round(ms, 4), tflops=round(flops / (ms * 1e-3) / 1e12, 1))
    return res


def _shader_clock_mhz():
    """The current shader clock as the driver's sysfs table marks it (MHz), None when unreadable.  Where the host
    shows several cards, the busy one is the one with the highest clock (idle cards sit at their lowest level)."""
    import glob
    best = None
    for path in sorted(glob.glob('/sys/class/drm/card*/device/pp_dpm_sclk')):
        try:
            for line in open(path):
                if line.rstrip().endswith('*'):
                    mhz = int(line.split(':')[1].strip().lower().split('mhz')[0])
                    best = mhz if best is None or mhz > best else best
        except (OSError, ValueError, IndexError):
            continue
    return best


def operand_pattern_leg(w, inp):
    """The three grouped products of this workload's shapes through the shipped kernel, one second of
    back-to-back launches each, with operands drawn as the workload draws them (N(0,1) activations, N(0,0.02)
    weights), all zero, and all one.  The instruction stream, the addresses and the memory traffic are the same
    in the three cases; only the switching activity of the operands differs, so the spread is what the power
    limit takes.  The shader clock is sampled from sysfs while the launches run."""
    import threading

    import torch

    from megablocks_amd import grouped_gemm_util as gg

    dev = torch.device('cuda', 0)
    if w.routing == 'router':
        logits = inp['x'].to(dev).float() @ inp['router_weight'].to(dev).float().t()
        top = logits.topk(w.top_k, dim=-1).indices
    else:
        top = inp['top_experts'].to(dev)
    sizes = torch.bincount(top.flatten(), minlength=w.experts).to(torch.int64)
    rows = int(sizes.sum())
    flops = 2.0 * rows * w.hidden * w.ffn
    res = {'what': 'mbx_gmm on this workload\'s shapes, >= 1 s of back-to-back launches per case', 'cases': {}}
    for pattern in ('workload', 'zeros', 'ones'):
        def draw(*shape, scale=1.0):
            if pattern == 'zeros':
                return torch.zeros(*shape, device=dev, dtype=w.dtype)
            if pattern == 'ones':
                return torch.ones(*shape, device=dev, dtype=w.dtype)
            return (torch.randn(*shape, device=dev) * scale).to(w.dtype)
        a, mid = draw(rows, w.hidden), draw(rows, w.ffn)
        w1 = draw(w.experts, w.ffn, w.hidden, scale=0.02)
        case = {}
        for name, fn in (('gmm_nt', lambda: gg.backend.gmm(a, w1, sizes, trans_b=True)),
                         ('gmm_nn', lambda: gg.backend.gmm(mid, w1, sizes)),
                         ('gmm_tn', lambda: gg.backend.gmm(mid, a, sizes, trans_a=True))):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            clocks, stop = [], threading.Event()

            def sample():
                while not stop.is_set():
                    mhz = _shader_clock_mhz()
                    if mhz:
                        clocks.append(mhz)
                    stop.wait(0.05)
            th = threading.Thread(target=sample)
            th.start()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            n, t0 = 0, time.perf_counter()
            e0.record()
            while time.perf_counter() - t0 < 1.0:
                for _ in range(20):
                    fn()
                n += 20
                torch.cuda.synchronize()
            e1.record()
            torch.cuda.synchronize()
            stop.set()
            th.join()
            ms = e0.elapsed_time(e1) / n
            case[name] = dict(avg_ms=round(ms, 4), tflops=round(flops / (ms * 1e-3) / 1e12, 1),
                              shader_clock_mhz=round(sum(clocks) / len(clocks)) if clocks else None)
        res['cases'][pattern] = case
        del a, mid, w1
    return res


def tile_ticks_leg(w, inp):
    """Where the time of an output tile goes, for the three grouped products of this workload's shapes: the kernels of
    libmbx_ticks.so (the library compiled with -DMBX_TICKS; loaded instead of libmbx.so by this leg) stamp every tile
    with the constant-rate clock (100 MHz) when it starts, when its first K tile has landed, after its last MFMA, after
    its last store has been issued and after the workgroup's LDS has been handed on.  One launch per product is read
    back; times are microseconds per tile, averaged over the launch's tiles."""
    import ctypes

    import torch

    from megablocks_amd import _lib
    from megablocks_amd import grouped_gemm_util as gg

    if not hasattr(_lib.lib, 'mbx_debug_set_ticks'):
        raise RuntimeError('bench.py --tile-ticks needs megablocks_amd/libmbx_ticks.so (python megablocks_amd/build.py)')
    set_ticks = _lib.lib.mbx_debug_set_ticks
    set_ticks.restype, set_ticks.argtypes = ctypes.c_int, [ctypes.c_void_p]
    dev = torch.device('cuda', 0)
    if w.routing == 'router':
        logits = inp['x'].to(dev).float() @ inp['router_weight'].to(dev).float().t()
        top = logits.topk(w.top_k, dim=-1).indices
    else:
        top = inp['top_experts'].to(dev)
    sizes = torch.bincount(top.flatten(), minlength=w.experts).to(torch.int64)
    rows = int(sizes.sum())
    a = torch.randn(rows, w.hidden, device=dev).to(w.dtype)
    mid = torch.randn(rows, w.ffn, device=dev).to(w.dtype)
    w1 = (torch.randn(w.experts, w.ffn, w.hidden, device=dev) * 0.02).to(w.dtype)
    workgroups, tiles, ids = 16384, 64, 8                               # kTickWorkgroups, kTickTiles, kTickIds of gmm_dma.h
    buf = torch.zeros(workgroups * tiles * ids, dtype=torch.int64, device=dev)
    res = {'what': 'per-tile phase times (us) from the time stamps of libmbx_ticks.so, one launch per product', 'products': {}}
    for name, fn in (('gmm_nt', lambda: gg.backend.gmm(a, w1, sizes, trans_b=True)),
                     ('gmm_nn', lambda: gg.backend.gmm(mid, w1, sizes)),
                     ('gmm_tn', lambda: gg.backend.gmm(mid, a, sizes, trans_a=True))):
        _lib.check(set_ticks(None), 'set_ticks')
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        buf.zero_()
        torch.cuda.synchronize()
        _lib.check(set_ticks(ctypes.c_void_p(buf.data_ptr())), 'set_ticks')
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        _lib.check(set_ticks(None), 'set_ticks')
        t = buf.view(workgroups, tiles, ids).cpu().double() / 100.0     # microseconds
        done = (t[:, :, 0] > 0) & (t[:, :, 1] > 0) & (t[:, :, 5] > 0)
        n = int(done.sum())
        phase = lambda x, y: float((t[:, :, y] - t[:, :, x])[done].mean())
        nxt = torch.zeros_like(done)
        nxt[:, :-1] = done[:, :-1] & done[:, 1:]
        between = (t[:, 1:, 0] - t[:, :-1, 5])[nxt[:, :-1]]
        start = t[:, :, 0][done].min()
        # a workgroup's first tile has no stores of a tile before it in flight; its last one may be a part of a tile
        # (mbx_gmm_ws: the tail of an NN launch) whose "stores" include the reduction of the parts
        per_ordinal = {}
        for o in range(min(tiles, 8)):
            if int(done[:, o].sum()):
                sel = done[:, o]
                per_ordinal[str(o)] = [round(float((t[:, o, y] - t[:, o, x])[sel].mean()), 2) for x, y in ((0, 1), (1, 2), (2, 4))]
        res['products'][name] = dict(
            launch_ms=round(e0.elapsed_time(e1), 4), tiles=n, workgroups=int(done.any(dim=1).sum()),
            start_to_first_k_tile=round(phase(0, 1), 2),
            of_which=dict(find_the_tile=round(phase(0, 6), 2), request_first_k_tiles=round(phase(6, 7), 2),
                          clear_accumulators=round(phase(7, 3), 2), wait_for_first_k_tile=round(phase(3, 1), 2)),
            main_loop=round(phase(1, 2), 2),
            last_mfma_to_last_store_issued=round(phase(2, 4), 2), hand_over=round(phase(4, 5), 2),
            between_tiles_of_a_workgroup=round(float(between.mean()), 2) if between.numel() else None,
            tile_total=round(phase(0, 5), 2), by_ordinal_of_the_tile_in_its_workgroup_start_loop_store=per_ordinal,
            first_tile_start_to_last_tile_end_ms=round(float(t[:, :, 5][done].max() - start) / 1000.0, 4))
    return res


def mfma_ceiling_leg():
    """A loop of matrix-core instructions alone (libmbx_probe.so: operands and accumulators stay in registers; no LDS
    reads, no memory traffic), about a second per case, on operands that are all zero, all one, and N(0,1) bf16
    values, for the 32x32x16 instruction the grouped GEMM uses and for 16x16x32.  The shader clock is measured inside
    the kernel (cycle counter against the 100 MHz wall clock).  On values that switch few bits the loop runs at the
    nominal peak; on random values the power limit lowers the clock, and what is left is the most any bf16 kernel
    can show on such data."""
    import ctypes

    import torch

    lib = ctypes.CDLL(os.path.join(ROOT, 'megablocks_amd', 'libmbx_probe.so'))
    lib.mbx_probe_mfma.restype = ctypes.c_int
    lib.mbx_probe_mfma.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                   ctypes.c_void_p, ctypes.c_void_p]
    dev = torch.device('cuda', 0)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    blocks = cus                                   # one workgroup of four waves per compute unit: one wave per SIMD
    n_vec = 1 << 16
    sink = torch.empty(blocks * 256, dtype=torch.float32, device=dev)
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    res = {'what': 'MFMA-only loop, one wave per SIMD on every compute unit, operands in registers', 'blocks': blocks, 'cases': {}}
    for kind, kname in ((0, 'mfma_32x32x16_bf16'), (1, 'mfma_16x16x32_bf16')):
        for pattern in ('zeros', 'ones', 'normal'):
            if pattern == 'zeros':
                ops = torch.zeros(n_vec * 8, dtype=torch.bfloat16, device=dev)
            elif pattern == 'ones':
                ops = torch.ones(n_vec * 8, dtype=torch.bfloat16, device=dev)
            else:
                ops = torch.randn(n_vec * 8, device=dev, generator=torch.Generator(device=dev).manual_seed(0)).to(torch.bfloat16)

            def launch(iters):
                rc = lib.mbx_probe_mfma(ops.data_ptr(), n_vec, kind, blocks, iters, sink.data_ptr(), clocks.data_ptr(), stream)
                if rc:
                    raise RuntimeError(f'mbx_probe_mfma failed: {rc}')
            launch(2000)
            torch.cuda.synchronize()
            iters = 400000 if kind == 0 else 200000  # 512 (or 1024) matrix-core cycles per iteration: about 0.1 s per launch
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            launches = 10
            e0.record()
            for _ in range(launches):
                launch(iters)
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / launches
            flops = blocks * 4.0 * iters * (16 * 32768 if kind == 0 else 64 * 16384)   # 16 MFMAs of 32x32x16 or 64 of 16x16x32 per iteration
            cyc, wall = clocks.tolist()
            res['cases'][f'{kname}/{pattern}'] = dict(
                ms_per_launch=round(ms, 3), tflops=round(flops / (ms * 1e-3) / 1e12, 1),
                frac_of_mfma_peak=round(flops / (ms * 1e-3) / MFMA_PEAK['bf16'], 4),
                shader_clock_mhz=round(cyc / wall * 100.0) if wall else None)
    return res


def cpu_leg(args, w, inp_full):
    """The CPU formulation (oracle) of the same layer, fp32, forward+backward, on a bounded sample."""
    import torch

    import oracle
    from megablocks_amd import synthetic

    cores = min(os.cpu_count() or 1, int(os.environ.get('OMP_NUM_THREADS', os.cpu_count() or 1)))
    torch.set_num_threads(cores)
    # The whole workload (c3, the largest default, is about 17 s per step on the 16 host threads of a GPU box, 70 s
    # for the four steps); a workload beyond 2.5e13 FLOP per step would be cut to half of its tokens (all experts and
    # their full weights either way: the work per token is unchanged); --cpu-tokens overrides.
    if args.cpu_tokens:
        T = args.cpu_tokens
    else:
        T = w.tokens if w.gemm_flops() <= 2.5e13 else w.tokens // 2
    inp = inp_full if T == w.tokens else synthetic.make_inputs(w, tokens=T, seed=0)
    act = w.activation()

    def step():
        x = inp['x'].clone().requires_grad_(True)
        rw = inp['router_weight'].clone().requires_grad_(True)
        w1, w2 = inp['w1'].requires_grad_(True), inp['w2'].requires_grad_(True)
        v1 = None if inp['v1'] is None else inp['v1'].requires_grad_(True)
        for p in (w1, w2, v1):
            if p is not None:
                p.grad = None
        if w.routing == 'router':
            _, ew, te = oracle.router_forward(x, rw, w.top_k, w.normalize)
        else:
            ew, te = inp['expert_weights'].clone().requires_grad_(True), inp['top_experts']
        out, _ = oracle.dmoe_forward(x, ew, te, w1, w2, v1, num_experts=w.experts, top_k=w.top_k, activation=act)
        out.backward(inp['grad'])

    step()  # warm-up
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    t = statistics.median(times)
    return dict(value=round(T / t, 1), unit='tokens/s', cores=cores, kind='port',
                sample=f'{T} of {w.tokens} tokens of workload {w.name}, fp32, fwd+bwd, 1 warm-up + 3 timed steps '
                       f'(median {t:.2f} s), torch {torch.get_num_threads()} threads',
                seconds_per_step=round(t, 3))


def main():
    args = parse()
    if args.gpus != 1:
        print(f'bench.py: this build runs on one GPU holding all experts; --gpus {args.gpus} is not supported '
              '(the expert-parallel all-to-all is out of scope).', file=sys.stderr)
        sys.exit(2)
    if args.tile_ticks:   # before the package is imported: it loads the library named here
        os.environ['MBX_LIBRARY'] = os.path.join(ROOT, 'megablocks_amd', 'libmbx_ticks.so')
    import torch

    from megablocks_amd import synthetic

    w = synthetic.WORKLOADS[args.config]
    if args.tokens:
        import dataclasses
        w = dataclasses.replace(w, tokens=args.tokens)
    inp = synthetic.make_inputs(w, seed=0)
    if args.tile_ticks:
        print(json.dumps({'config': {'workload': f'{w.name}: {w.description}', 'tokens': w.tokens},
                          'tile_ticks': tile_ticks_leg(w, inp)}))
        return
    ms_per_step, ms_wall, agg, layer = gpu_leg(args, w, inp)

    slots_scale = 1.0
    if w.mlp_impl == 'sparse':
        # every gmm record carries the padded row count the kernels were handed
        any_gmm = next(d for n, d in agg.items() if n.startswith('gmm'))
        slots_scale = w.slots / float(any_gmm['meta']['rows'])
    gemm, perm = summarize(w, agg, slots_scale)

    dn = dtype_name(w.dtype)
    gemm_ms = sum(g['avg_ms'] * g['launches'] for g in gemm.values()) / args.steps
    perm_ms = sum(p['avg_ms'] * p['launches'] for p in perm.values()) / args.steps
    dom_name, dom = max(gemm.items(), key=lambda kv: kv[1]['avg_ms'] * kv[1]['launches'])
    # The kernel is bound by whichever roofline its arithmetic intensity puts lower (the ridge of the part is
    # MFMA peak / HBM peak = 312 FLOP per byte in bf16): c2's 256-row experts stream their weights.
    traffic, traffic_source = measured_traffic(w.name if not args.tokens else None, dom_name)
    if dom['flops_per_launch'] / dom['bytes_per_launch'] >= MFMA_PEAK[dn] / HBM_PEAK:
        roofline = dict(bound='mfma', kernel=dom_name, achieved=dom['tflops'], peak=MFMA_PEAK[dn] / 1e12, unit='TFLOP/s',
                        frac=dom['frac_of_mfma_peak'], traffic=traffic, traffic_source=traffic_source,
                        algorithmic_bytes_per_launch=dom['bytes_per_launch'],
                        flops_per_launch=dom['flops_per_launch'], avg_launch_ms=dom['avg_ms'])
    else:
        roofline = dict(bound='hbm', kernel=dom_name, achieved=dom['gbps'], peak=HBM_PEAK / 1e9, unit='GB/s',
                        frac=dom['frac_of_hbm_peak'], traffic=traffic, traffic_source=traffic_source,
                        bytes_per_launch=dom['bytes_per_launch'], avg_launch_ms=dom['avg_ms'])
    step_flops = w.gemm_flops()
    if args.forward_only:
        step_flops = sum(g['flops_per_launch'] * g['launches'] for g in gemm.values()) / args.steps
    all_gemm_tflops = step_flops / (gemm_ms * 1e-3) / 1e12 if gemm_ms else None

    out = {
        'metric': 'dmoe_layer_fwd_tokens_per_s' if args.forward_only else 'dmoe_layer_fwd_bwd_tokens_per_s',
        'value': round(w.tokens / (ms_per_step * 1e-3), 1),
        'unit': 'tokens/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': round(ms_per_step, 4),
        'ms_per_step_wall': round(ms_wall, 4),
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': dn,
        'data': 'synthetic',
        'config': {'workload': f'{w.name}: {w.description}', 'tokens': w.tokens, 'hidden': w.hidden, 'ffn': w.ffn,
                   'experts': w.experts, 'top_k': w.top_k, 'mlp_type': w.mlp_type, 'mlp_impl': w.mlp_impl,
                   'routing': w.routing, 'memory_optimized_mlp': args.memory_optimized, 'graph_replay': args.graph},
        'roofline': roofline,
        'gemm': {'ms_per_step': round(gemm_ms, 4), 'tflops_all_launches': round(all_gemm_tflops, 1),
                 'frac_of_mfma_peak': round(all_gemm_tflops * 1e12 / MFMA_PEAK[dn], 4), 'kernels': gemm},
        'permute': {'ms_per_step': round(perm_ms, 4), 'kernels': perm},
    }
    if args.library_gemm:
        out['library_gemm'] = library_gemm_leg(w, inp)
    if args.operand_patterns:
        out['operand_patterns'] = operand_pattern_leg(w, inp)
    if args.mfma_ceiling:
        out['mfma_ceiling'] = mfma_ceiling_leg()
    if not args.no_cpu and not args.forward_only:
        del layer
        torch.cuda.empty_cache()
        out['cpu_baseline'] = cpu_leg(args, w, inp)
    else:
        out['cpu_baseline'] = None
    print(json.dumps(out))


if __name__ == '__main__':
    main()
