#!/usr/bin/env python3
"""Benchmark of the MI355X fake-quantization path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]

One step = one pass of the MX block-scaling workload (BASELINE configs[1]) over an 8192 x 8192 bf16 tensor
resident in HBM -- 1 x 32 blocks, power-of-two (E8M0) shared scale, elements cast to E4M3, E5M2 and E2M3 -- plus one
MoR 128 x 128 pass over an 8192 x 8192 N(0,1) tensor (four launches).  The launches rotate over several input /
output buffer pairs, so that every byte comes from HBM and not from the 256 MB last-level cache.  The printed JSON
line reports algorithmic HBM GB/s (2 B read + 2 B written per element + 4 B of meta per block where the op returns
meta) for the whole step, the roofline fraction of the kernel furthest below the roofline from HIP events recorded
around its launches in the timed region (with the cache-warm figure of every kernel beside it), the roofline
fraction of every BASELINE configuration from HBM (`roofline.per_config`), what bounds the MoR kernel
(`roofline.mor_128x128_breakdown`), the clocks and the power over the first milliseconds after idle
(`after_idle_transient`), the other configurations, and the CPU oracle timed on bounded samples of the same workloads
on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the other configurations")
    ap.add_argument("--no-warm", action="store_true", help="skip the same-buffer (cache-warm) and plain-copy side measurements")
    ap.add_argument("--rotate", type=int, default=6, help="input / output buffer pairs the timed launches rotate over")
    ap.add_argument("--preheat-ms", type=float, default=40.0,
                    help="untimed steps run for this long before the warmup, so that the GPU's clocks have left their idle state (0: none)")
    ap.add_argument("--rows", type=int, default=8192)
    ap.add_argument("--cols", type=int, default=8192)
    return ap.parse_args()


def gen_c2_gpu(torch, rows, cols, seed=1002):
    """Student-t(3) * 0.02 with 0.1 % of the elements x1000, generated on the GPU."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    z = torch.randn(rows, cols, device="cuda", generator=g)
    d = torch.zeros(rows, cols, device="cuda")
    for _ in range(3):
        d += torch.randn(rows, cols, device="cuda", generator=g) ** 2
    t = z / torch.sqrt(d / 3) * 0.02
    mask = torch.rand(rows, cols, device="cuda", generator=g) < 1e-3
    return torch.where(mask, t * 1000, t).to(torch.bfloat16).contiguous()


def gen_c4_gpu(torch, rows, cols, seed=1004, tile=128):
    g = torch.Generator(device="cuda").manual_seed(seed)
    gy, gx = (rows + tile - 1) // tile, (cols + tile - 1) // tile
    u = torch.rand(gy, gx, device="cuda", generator=g)
    kind = torch.where(u < 0.7, 0, torch.where(u < 0.9, 1, 2)).repeat_interleave(tile, 0).repeat_interleave(tile, 1)[:rows, :cols]
    t = torch.randn(rows, cols, device="cuda", generator=g)
    sign = torch.where(torch.rand(rows, cols, device="cuda", generator=g) < 0.5, -1.0, 1.0)
    t = torch.where(kind == 1, torch.exp(3 * t) * sign, torch.where(kind == 2, t * 1e-4, t))
    return t.to(torch.bfloat16).contiguous()


class Launcher:
    """Thin caller of the C ABI on torch's current stream."""

    def __init__(self, torch, cabi):
        self.torch, self.cabi, self.L = torch, cabi, cabi.lib()

    def stream(self):
        return self.torch.cuda.current_stream().cuda_stream

    def fake_quantize(self, x, out, meta, br, bc, clamp, mode, sf, flags=0):
        r, c = x.shape
        self.cabi.check(self.L.mor_fake_quantize(x.data_ptr(), out.data_ptr(), meta.data_ptr(), r, c, br, bc,
                                                 float(clamp), mode, sf, flags, self.stream()))

    def block_format(self, x, out, br, bc, fmt, sf, flags=0):
        r, c = x.shape
        self.cabi.check(self.L.mor_block_format(x.data_ptr(), out.data_ptr(), r, c, br, bc, fmt, sf, flags, self.stream()))


    def scaling_state(self, rows, cols, br, bc, channel):
        """Scalar outputs and the workspace of one mor_block_scaling call (allocated once, outside the timed region)."""
        t = self.torch
        op = self.cabi.OP_CHANNEL_SCALING if channel else self.cabi.OP_BLOCK_SCALING
        nbytes = self.L.mor_workspace_bytes(op, rows, cols, br, bc)
        return {"meta": t.empty(1, dtype=t.int32, device="cuda"), "amax": t.empty(1, dtype=t.float32, device="cuda"),
                "nnz": t.empty(1, dtype=t.int32, device="cuda"), "err": t.empty(1, dtype=t.float32, device="cuda"),
                "ws": t.empty(max(nbytes, 4), dtype=t.uint8, device="cuda"), "nbytes": nbytes, "channel": int(channel)}

    def block_scaling(self, x, out, st, br, bc, thr, ss_mode):
        r, c = x.shape
        self.cabi.check(self.L.mor_block_scaling(x.data_ptr(), out.data_ptr(), st["meta"].data_ptr(), st["amax"].data_ptr(),
                                                 st["nnz"].data_ptr(), st["err"].data_ptr(), r, c, br, bc, float(thr), ss_mode,
                                                 st["channel"], st["ws"].data_ptr(), st["nbytes"], 0, self.stream()))


def time_launches(torch, fn, steps, warmup):
    """-> (mean ms per launch from one pair of HIP events around `steps` back-to-back launches, wall ms per launch)"""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return a.elapsed_time(b) / steps, wall


def read_traffic(kernel):
    """-> (HBM bytes per launch of `kernel`, where the figure comes from).  Hardware counters cannot be read from inside
    the run: the figure is the one in the committed counter summary (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
    script, each scaled by the same counter's reading for the library's plain copy kernel); None when it holds none."""
    rel = os.path.join("profiles", "bench_step_mx_1x32_and_mor_128x128_8192x8192_hbm_traffic.txt")
    try:
        for line in open(os.path.join(ROOT, rel)):
            f = line.split()
            if len(f) >= 3 and f[0] == "traffic_bytes" and f[1] == kernel:
                return int(f[2]), rel + " (rocprofv3 --pmc, not measured in this run)"
    except OSError:
        pass
    return None, None


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: every quantization block is independent, so more GPUs only shard rows; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import importlib.util
    spec = importlib.util.spec_from_file_location("mor_amd_build", os.path.join(ROOT, "mor_amd", "build.py"))
    build_mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build_mod)
    build_mod.ensure_built()                # nothing to do when the libraries travelled with the tree
    import torch
    from mor_amd import _cabi
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP library has no CPU path)", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    run = Launcher(torch, _cabi)
    rows, cols = args.rows, args.cols
    K, W = args.steps, args.warmup

    # Inputs and outputs of the timed step, ROT copies of each so that no launch finds its data in the 256 MB last-level
    # cache: the MX tensor (Student-t, outliers) and the MoR tensor (N(0,1)), both rows x cols bf16.
    ROT = args.rotate
    x_mx = gen_c2_gpu(torch, rows, cols)
    g = torch.Generator(device="cuda").manual_seed(1001)
    x_mor = torch.randn(rows, cols, device="cuda", generator=g).to(torch.bfloat16)
    xs_mx = [x_mx] + [x_mx.clone() for _ in range(ROT - 1)]
    xs_mor = [x_mor] + [x_mor.clone() for _ in range(ROT - 1)]
    outs = [torch.empty_like(x_mx) for _ in range(ROT)]
    meta = torch.empty((rows, cols // 32), dtype=torch.int32, device="cuda")
    meta_mor = torch.empty(((rows + 127) // 128, (cols + 127) // 128), dtype=torch.int32, device="cuda")
    nelem = rows * cols
    nblocks = nelem // 32
    launches = [
        ("mx_e4m3", lambda i: run.fake_quantize(xs_mx[i], outs[i], meta, 1, 32, 0.0, 2, 2), nelem * 4 + nblocks * 4),
        ("mx_e5m2", lambda i: run.fake_quantize(xs_mx[i], outs[i], meta, 1, 32, 0.0, 3, 2), nelem * 4 + nblocks * 4),
        ("mx_e2m3", lambda i: run.block_format(xs_mx[i], outs[i], 1, 32, _cabi.FMT_E2M3, 2), nelem * 4),
        ("mor_128x128", lambda i: run.fake_quantize(xs_mor[i], outs[i], meta_mor, 128, 128, 1e-15, 1, 1), nelem * 4 + meta_mor.numel() * 4),
    ]
    bytes_per_step = sum(b for _, _, b in launches)

    turn = [0]

    def rotating(fn):
        turn[0] = (turn[0] + 1) % ROT
        fn(turn[0])

    def timed_groups(k):
        """k launches of each kernel, grouped by kernel, one HIP-event pair per group -> ([ms per launch], wall ms per step)"""
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(len(launches) + 1)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        marks[0].record()
        for i, (_, fn, _) in enumerate(launches):
            for _ in range(k):
                rotating(fn)
            marks[i + 1].record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / k
        return [marks[i].elapsed_time(marks[i + 1]) / k for i in range(len(launches))], wall

    # In the first 15 ms of load after the GPU has been idle the MoR kernel, the one with the most arithmetic, goes
    # through a transient: 48-49 us per launch at the start, 52-54 us between 3 and 6 ms, 47 us from 15 ms on, where it
    # stays (after_idle_transient below records it with the shader clock and the power; the MX kernels stay at 42-44 us
    # throughout).  A measurement of 20 steps right after 5 warmup steps sits in the middle of it.  Those first 20 steps
    # are timed for the record, and then untimed steps run for --preheat-ms before the W warmup steps: the timed region
    # measures the sustained rate.
    for _, fn, _ in launches:               # (the very first launch of a kernel also loads its code: not part of any figure)
        rotating(fn)
    first_ms, first_wall = timed_groups(20)
    preheat_steps = 0
    if args.preheat_ms > 0:
        t_end = time.perf_counter() + args.preheat_ms * 1e-3
        while time.perf_counter() < t_end:
            for _ in range(8):
                for _, fn, _ in launches:
                    rotating(fn)
            torch.cuda.synchronize()
            preheat_steps += 8
    for _ in range(W):
        for _, fn, _ in launches:
            rotating(fn)
    torch.cuda.synchronize()
    # The timed region holds exactly K steps of work.  Its launches are grouped by kernel (K x E4M3, K x E5M2,
    # K x E2M3, K x MoR) so that one pair of HIP events brackets the K launches of each kernel: an event between every
    # two launches would add its own few microseconds to 45-microsecond kernels.  Events and launches share torch's
    # current stream.
    group_ms, ms_per_step = timed_groups(K)
    value = bytes_per_step / (ms_per_step * 1e-3) / 1e9

    def rate(nbytes, ms):
        return {"ms": round(ms, 5), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1), "frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    per_kernel = {}
    for i, (name, fn, nbytes) in enumerate(launches):
        per_kernel[name] = dict(rate(nbytes, group_ms[i]), bytes=nbytes)
        per_kernel[name]["first_20_steps_after_idle"] = rate(nbytes, first_ms[i])
    # The same kernels on one buffer pair, launch after launch: the 268 MB working set is then about the size of the
    # last-level cache, which serves part of it -- reported beside the HBM figure, never as it.  And the library's plain
    # copy over the same rotation: what the memory system gives a kernel that only moves the bytes.
    if not args.no_warm:
        for name, fn, nbytes in launches:
            ms = time_launches(torch, lambda: fn(0), max(K, 20), 3)[0]
            per_kernel[name]["same_buffers_warm_cache"] = rate(nbytes, ms)
        copy_ms = time_launches(torch, lambda: rotating(lambda i: run.fake_quantize(xs_mx[i], outs[i], meta_mor, 128, 128, 0.0, 7, 1)), max(K, 20), 3)[0]
        per_kernel["plain_copy_mode7"] = dict(rate(nelem * 4 + meta_mor.numel() * 4, copy_ms), bytes=nelem * 4 + meta_mor.numel() * 4,
                                              note="not part of the step: the library's bf16 copy over the same rotating buffers")
    timed = [n for n, _, _ in launches]
    dom = min(timed, key=lambda n: per_kernel[n]["frac"])
    traffic, traffic_src = read_traffic(dom)
    roofline = {"bound": "hbm", "kernel": dom, "achieved": per_kernel[dom]["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": per_kernel[dom]["frac"], "traffic": traffic, "traffic_source": traffic_src,
                "buffers": f"{ROT} input / output pairs in rotation ({ROT * 2 * nelem * 2 / 2**30:.1f} GiB): nothing is cache-resident",
                "per_kernel": per_kernel}
    x = x_mx
    del xs_mx, xs_mor, outs

    transient = None
    extra = {}
    if not args.no_extra:
        roofline["per_config"] = per_config_from_hbm(torch, run, _cabi, per_kernel, rows, cols)
        roofline["mor_128x128_breakdown"] = mor_breakdown(torch, run, _cabi, rows, cols)
        transient = after_idle_transient(torch, run, rows, cols)
        extra = other_configs(torch, run, _cabi, max(5, K // 2), max(2, W // 2))
        c5 = extra.get("c5_llama3_8b_layer", {})
        for fam in ("mor_128x128", "block_e4m3_128x128", "per_channel_rows_and_columns"):
            if fam in c5:
                roofline["per_config"]["c5_llama3_8b_layer_" + fam] = {k: c5[fam][k] for k in ("total_ms", "total_GB", "GBps", "frac")}

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(torch, x, x_mor)

    line = {
        "metric": "fake-quant HBM GB/s (rd+wr), MX 1x32 E8M0 block scaling (E4M3+E5M2+E2M3) and MoR 128x128 on 8192x8192 bf16",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"configs[1]: MX block scaling {rows}x{cols} bf16, 1x32 blocks, E8M0 scale, E4M3+E5M2+E2M3, "
                               f"plus MoR 128x128 (fp32 scale, error criterion) on a {rows}x{cols} N(0,1) tensor, per step; "
                               f"{ROT} buffer pairs in rotation",
                   "arithmetic": "bf16 tensors, fp32 / integer arithmetic, gfx950 fp8 / fp6 converts",
                   "preheat": f"{preheat_steps} untimed steps ({args.preheat_ms:g} ms) before the {W} warmup steps: between 2 and 8 ms of load after idle the "
                              f"MoR kernel runs up to a tenth slower (after_idle_transient: per-batch times with the shader clock and the power beside "
                              f"them -- the clock stays within 4 % of 2.4 GHz throughout, the power sensor climbs from 300 W to 700 W over 60 ms); the "
                              f"first 20 steps after idle took {first_wall:.5f} ms each (per kernel: first_20_steps_after_idle), the timed steps are "
                              f"the sustained rate",
                   "elements_per_s": round(4 * nelem / (ms_per_step * 1e-3), 0), "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4)},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "after_idle_transient": transient,
        "other_configs": extra,
    }
    print(json.dumps(line))


def cold_launches(torch, make_fn, nbufs, target_ms=10.0, preheat_ms=30.0):
    """ms per launch of fn(i), i rotating over nbufs buffer sets (so that nothing is found in the last-level cache),
    over about target_ms of back-to-back launches after preheat_ms of untimed ones."""
    fn = make_fn
    i = 0
    t_end = time.perf_counter() + preheat_ms * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(8):
            fn(i % nbufs)
            i += 1
        torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(10):
        fn(i % nbufs)
        i += 1
    b.record()
    torch.cuda.synchronize()
    n = max(10, min(2000, int(target_ms / (a.elapsed_time(b) / 10))))
    a.record()
    for _ in range(n):
        fn(i % nbufs)
        i += 1
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / n


def rate_of(nbytes, nelem, ms):
    return {"ms": round(ms, 5), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1), "frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "elements_per_s": round(nelem / (ms * 1e-3), 0), "bytes": nbytes}


def per_config_from_hbm(torch, run, cabi, per_kernel, rows, cols):
    """Every BASELINE configuration with its data coming from HBM: tensors smaller than the 256 MB last-level cache
    rotate over 6 buffer pairs.  C2 and MoR on the benchmark tensor are the timed step's own figures; C5 is added by
    the layer sweep (its tensors are 8 to 470 MB each and follow one another)."""
    res = {}
    NB = 6
    for k in ("mx_e4m3", "mx_e5m2", "mx_e2m3"):
        res["c2_" + k + f"_{rows}x{cols}"] = {kk: per_kernel[k][kk] for kk in ("ms", "GBps", "frac", "bytes")}
    res[f"mor_128x128_{rows}x{cols}_normal"] = {kk: per_kernel["mor_128x128"][kk] for kk in ("ms", "GBps", "frac", "bytes")}
    # C1: per-tensor E4M3 on 4096 x 4096 N(0,1): with the caller's scale (one pass, 4 B/element) and with the tensor amax
    # found on the GPU (block-scaling op, ss_mode 4: two reads and a write, 6 B/element)
    g = torch.Generator(device="cuda").manual_seed(1001)
    x1 = torch.randn(4096, 4096, device="cuda", generator=g).to(torch.bfloat16)
    xs = [x1] + [x1.clone() for _ in range(NB - 1)]
    outs = [torch.empty_like(x1) for _ in range(NB)]
    m1 = torch.empty((32, 32), dtype=torch.int32, device="cuda")
    scale = float(448.0 / x1.float().abs().max().item())
    n = x1.numel()
    res["c1_per_tensor_e4m3_4096x4096_callers_scale"] = rate_of(n * 4, n, cold_launches(torch, lambda i: run.fake_quantize(xs[i], outs[i], m1, 128, 128, scale, 4, 1), NB))
    st1 = run.scaling_state(4096, 4096, 128, 128, False)
    res["c1_per_tensor_e4m3_4096x4096_gpu_amax_ss4"] = rate_of(n * 6, n, cold_launches(torch, lambda i: run.block_scaling(xs[i], outs[i], st1, 128, 128, 0.045, 4), NB))
    res["c1_per_tensor_e4m3_4096x4096_gpu_amax_ss4"]["note"] = "three dependent launches on a 32 MiB tensor; 6 B/element (4 B/element: frac x 2/3)"
    del xs, outs, x1
    # C3: per-row fp32 scale on the 16384 x 4096 weight matrix: fake_quantize (E4M3, E5M2) and the channel-scaling op the
    # reference's callers use (ss_mode 3; amax, non-zero count, error sum and the bf16 fallback decision included)
    g = torch.Generator(device="cuda").manual_seed(1003)
    w = torch.randn(16384, 4096, device="cuda", generator=g) * 0.02
    w[torch.randperm(16384, device="cuda", generator=g)[:164]] *= 100
    w[7] = 0
    w = w.to(torch.bfloat16)
    ws = [w] + [w.clone() for _ in range(NB - 1)]
    ows = [torch.empty_like(w) for _ in range(NB)]
    mw = torch.empty((16384, 1), dtype=torch.int32, device="cuda")
    n = w.numel()
    res["c3_per_row_e4m3_16384x4096"] = rate_of(n * 4 + 16384 * 4, n, cold_launches(torch, lambda i: run.fake_quantize(ws[i], ows[i], mw, 1, 4096, 0.0, 2, 1), NB))
    res["c3_per_row_e5m2_16384x4096"] = rate_of(n * 4 + 16384 * 4, n, cold_launches(torch, lambda i: run.fake_quantize(ws[i], ows[i], mw, 1, 4096, 0.0, 3, 1), NB))
    st3 = run.scaling_state(16384, 4096, 1, 4096, True)
    res["c3_per_row_e4m3_16384x4096_channel_op_ss3"] = rate_of(n * 4, n, cold_launches(torch, lambda i: run.block_scaling(ws[i], ows[i], st3, 1, 4096, 0.045, 3), NB))
    del ws, ows, w
    # C4: MoR 128 x 128 on the 16384 x 14336 tile mixture (470 MB: nothing of it is found in a cache)
    x4 = gen_c4_gpu(torch, 16384, 14336)
    o4 = torch.empty_like(x4)
    m4 = torch.empty((128, 112), dtype=torch.int32, device="cuda")
    n = x4.numel()
    res["c4_mor_128x128_16384x14336_mixture"] = rate_of(n * 4 + m4.numel() * 4, n, cold_launches(torch, lambda i: run.fake_quantize(x4, o4, m4, 128, 128, 1e-15, 1, 1), 1))
    torch.cuda.synchronize()
    hist = torch.bincount(m4.flatten(), minlength=13).tolist()
    res["c4_mor_128x128_16384x14336_mixture"]["meta_histogram"] = {str(i): h for i, h in enumerate(hist) if h}
    return res


def mor_breakdown(torch, run, cabi, rows, cols):
    """What bounds the MoR 128 x 128 kernel on the benchmark tensor, all from HBM (6 buffer pairs in rotation): the
    library's linear copy, a copy through the tile kernel's own walk (mor_block_format with MOR_FMT_COPY: every 128 x 128
    tile read, its amax found, written back unchanged), block E4M3 on the same tiles, and MoR on a tensor whose tiles
    are all decided by their range (no error pass) and on one whose tiles all take the error pass."""
    NB = 6
    g = torch.Generator(device="cuda").manual_seed(1001)
    base = torch.randn(rows, cols, device="cuda", generator=g)
    meta = torch.empty((rows // 128, cols // 128), dtype=torch.int32, device="cuda")
    n = rows * cols
    nb = n * 4 + meta.numel() * 4
    res = {}

    def bufs(t):
        t = t.to(torch.bfloat16)
        return [t] + [t.clone() for _ in range(NB - 1)]

    xs = bufs(base)
    outs = [torch.empty_like(xs[0]) for _ in range(NB)]
    res["linear_copy_mode7"] = rate_of(nb, n, cold_launches(torch, lambda i: run.fake_quantize(xs[i], outs[i], meta, 128, 128, 0.0, 7, 1), NB))
    res["tile_walk_copy_128x128"] = rate_of(n * 4, n, cold_launches(torch, lambda i: run.block_format(xs[i], outs[i], 128, 128, cabi.FMT_COPY, 1), NB))
    # the same copy through the same kernel (a block in a workgroup's registers, 8 vectors per lane) for blocks of other
    # shapes with as many elements: 2 whole rows (32 KiB that lie together: a linear copy in thick workgroups) and
    # 16 rows x 2 KiB; and for thin blocks of one row of 4096 elements (2 vectors per lane)
    for name, br, bc in (("block_walk_copy_2x8192", 2, 8192), ("block_walk_copy_16x1024", 16, 1024), ("block_walk_copy_1x4096", 1, 4096)):
        if rows % br == 0 and cols % bc == 0:
            res[name] = rate_of(n * 4, n, cold_launches(torch, lambda i: run.block_format(xs[i], outs[i], br, bc, cabi.FMT_COPY, 1), NB))
    res["block_e4m3_128x128"] = rate_of(nb, n, cold_launches(torch, lambda i: run.fake_quantize(xs[i], outs[i], meta, 128, 128, 0.0, 2, 1), NB))
    res["mor_normal_data"] = rate_of(nb, n, cold_launches(torch, lambda i: run.fake_quantize(xs[i], outs[i], meta, 128, 128, 1e-15, 1, 1), NB))
    torch.cuda.synchronize()
    del xs
    xs = bufs(torch.sign(base) * (base.abs() + 0.02))            # amax / amin of every tile below 114688: E4M3 by range
    res["mor_every_tile_decided_by_range"] = rate_of(nb, n, cold_launches(torch, lambda i: run.fake_quantize(xs[i], outs[i], meta, 128, 128, 1e-15, 1, 1), NB))
    del xs
    t = base.clone()
    t[::128, ::128] = 1e-6                                       # one tiny element per tile: every tile takes the error pass
    xs = bufs(t)
    del t
    res["mor_every_tile_takes_the_error_pass"] = rate_of(nb, n, cold_launches(torch, lambda i: run.fake_quantize(xs[i], outs[i], meta, 128, 128, 1e-15, 1, 1), NB))
    return res


def after_idle_transient(torch, run, rows, cols):
    """The first milliseconds of load after the GPU has been idle: 40 batches of 20 MoR launches (an event pair each) with
    the shader clock and the board power read from sysfs by a host thread meanwhile (pp_dpm_sclk, hwmon power1_input)."""
    import glob
    import threading
    dev = "/sys/class/drm/card0/device"
    power_files = glob.glob(dev + "/hwmon/*/power1_input")

    def read(path):
        try:
            with open(path) as f:
                return f.read()
        except OSError:
            return ""

    def sclk():
        for line in read(dev + "/pp_dpm_sclk").splitlines():
            if "*" in line:
                return line.split(":")[1].replace("*", "").strip()
        return None

    g = torch.Generator(device="cuda").manual_seed(1001)
    x = torch.randn(rows, cols, device="cuda", generator=g).to(torch.bfloat16)
    xs = [x] + [x.clone() for _ in range(5)]
    outs = [torch.empty_like(x) for _ in range(6)]
    meta = torch.empty((rows // 128, cols // 128), dtype=torch.int32, device="cuda")
    run.fake_quantize(xs[0], outs[0], meta, 128, 128, 1e-15, 1, 1)
    torch.cuda.synchronize()
    time.sleep(2.0)                                   # idle
    samples, stop = [], [False]

    def sampler():
        while not stop[0]:
            samples.append((time.perf_counter(), sclk(), read(power_files[0]).strip() if power_files else ""))

    th = threading.Thread(target=sampler)
    th.start()
    time.sleep(0.01)
    t0 = time.perf_counter()
    pairs = []
    for b in range(40):
        a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(20):
            run.fake_quantize(xs[(b * 20 + i) % 6], outs[(b * 20 + i) % 6], meta, 128, 128, 1e-15, 1, 1)
        e.record()
        pairs.append((a, e))
    torch.cuda.synchronize()
    stop[0] = True
    th.join()
    first = pairs[0][0]
    batches = [{"start_ms": round(first.elapsed_time(a), 2), "us_per_launch": round(a.elapsed_time(e) / 20 * 1e3, 2)} for a, e in pairs]
    series, last = [], None
    for t, s, p in samples:
        if (s, p) != last and t >= t0 - 0.005:
            series.append({"t_ms": round((t - t0) * 1e3, 2), "sclk": s, "power_W": round(int(p) / 1e6, 0) if p.isdigit() else None})
            last = (s, p)
    slow = max(batches, key=lambda b: b["us_per_launch"])
    return {"what": "MoR 128x128 launches back to back from an idle GPU, 20 per batch; sclk and power (the sensor's running average) from sysfs",
            "batches": batches, "slowest_batch": slow, "last_batch": batches[-1], "sclk_and_power": series[:40]}


def other_configs(torch, run, cabi, K, W):
    """Per-launch figures for the remaining configurations (HIP events around each launch)."""
    res = {}

    def add(name, fn, nbytes, nelem):
        ms, wall = time_launches(torch, fn, K, W)
        # short bursts after idle are not the sustained rate (clock ramp; the MoR kernels run 15 % slower between 2 and
        # 8 ms into a burst): 30 ms of untimed launches, then about 10 ms of timed ones
        ms, wall = time_launches(torch, fn, min(1000, max(K, int(10.0 / ms) + 1)), min(3000, int(30.0 / ms) + 1))
        res[name] = {"ms": round(ms, 5), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1), "frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "elements_per_s": round(nelem / (ms * 1e-3), 0)}

    # (every figure in this function is taken on one buffer pair, launch after launch; tensors of up to 128 MiB are then
    # partly served by the 256 MB last-level cache -- only the 16384 x 14336 cases are pure HBM figures)
    g = torch.Generator(device="cuda").manual_seed(1001)
    x = torch.randn(8192, 8192, device="cuda", generator=g).to(torch.bfloat16)
    out = torch.empty_like(x)
    meta = torch.empty((64, 64), dtype=torch.int32, device="cuda")
    n = x.numel()
    add("copy_mode7_8192x8192", lambda: run.fake_quantize(x, out, meta, 128, 128, 0.0, 7, 1), n * 4 + meta.numel() * 4, n)
    add("block_e4m3_128x128_8192x8192_fp32scale", lambda: run.fake_quantize(x, out, meta, 128, 128, 0.0, 2, 1), n * 4 + meta.numel() * 4, n)
    # blocks beyond the 16384 elements a 256-thread workgroup keeps in registers (same 67.1 M elements)
    add("block_e4m3_128x256_8192x8192", lambda: run.fake_quantize(x, out, meta, 128, 256, 0.0, 2, 1), n * 4, n)
    add("block_e4m3_256x256_8192x8192", lambda: run.fake_quantize(x, out, meta, 256, 256, 0.0, 2, 1), n * 4, n)
    add("mor_256x256_8192x8192_normal", lambda: run.fake_quantize(x, out, meta, 256, 256, 1e-15, 1, 1), n * 4, n)
    add("per_row_e4m3_2048x32768", lambda: run.fake_quantize(x.view(2048, 32768), out.view(2048, 32768), meta, 1, 32768, 0.0, 2, 1), n * 4, n)
    add("per_row_e4m3_512x131072", lambda: run.fake_quantize(x.view(512, 131072), out.view(512, 131072), meta, 1, 131072, 0.0, 2, 1), n * 4, n)
    # x and its transpose from one read, 128 x 128 tiles (one read + two writes: 6 B/element); the reference's callers
    # run the op on x and on x.t().contiguous(): two launches and a transposing copy, 12 B/element
    out_t = torch.empty_like(x)
    meta_t = torch.empty_like(meta)
    st_ = run.stream
    for mode, key in ((1, "dual_tiles_mor_128x128_8192x8192"), (2, "dual_tiles_e4m3_128x128_8192x8192")):
        add(key, lambda: cabi.check(run.L.mor_fake_quantize_dual_tiles(x.data_ptr(), out.data_ptr(), meta.data_ptr(), out_t.data_ptr(),
                                                                         meta_t.data_ptr(), 8192, 8192, 1e-15, mode, 1, st_())), n * 6, n)
    del out_t
    mor_tile_codes(torch, cabi, run, add, x, out, "8192x8192_normal")
    # E8M2 rounding (mor_e8mx): without a scale (one pass, 4 B/element) and with the tensor-amax strategy (a pass that
    # finds the amax, then the quantize pass: 6 B/element)
    nb8 = run.L.mor_workspace_bytes(cabi.OP_E8MX, 8192, 8192, 32, 32)
    ws8 = torch.empty(max(nb8, 4), dtype=torch.uint8, device="cuda")
    for strat, key, bpe in ((3, "e8m2_no_scale_8192x8192", 4), (1, "e8m2_tensor_amax_8192x8192", 6)):
        add(key, lambda: cabi.check(run.L.mor_e8mx(x.data_ptr(), out.data_ptr(), 8192, 8192, 32, 32, 2, strat, ws8.data_ptr(), nb8, 0, st_())), n * bpe, n)
    del ws8
    # C1: per-tensor E4M3, 4096x4096, scale from the tensor amax (the quantize pass only: 4 B/element)
    x1 = x[:4096, :4096].contiguous()
    o1 = torch.empty_like(x1)
    m1 = torch.empty((32, 32), dtype=torch.int32, device="cuda")
    scale = float(448.0 / x1.float().abs().max().item())
    add("c1_per_tensor_e4m3_4096x4096", lambda: run.fake_quantize(x1, o1, m1, 128, 128, scale, 4, 1), x1.numel() * 4, x1.numel())
    # C1 with the tensor amax found on the GPU: block-scaling op, ss_mode 4 (two reads + one write: 6 B/element)
    st1 = run.scaling_state(4096, 4096, 128, 128, False)
    add("c1_per_tensor_e4m3_4096x4096_gpu_amax_ss4", lambda: run.block_scaling(x1, o1, st1, 128, 128, 0.045, 4), x1.numel() * 6, x1.numel())
    del x, out, x1, o1
    # C3: per-row fp32 scale, 16384x4096
    g = torch.Generator(device="cuda").manual_seed(1003)
    w = torch.randn(16384, 4096, device="cuda", generator=g) * 0.02
    hot = torch.randperm(16384, device="cuda", generator=g)[:164]
    w[hot] *= 100
    w[7] = 0
    w = w.to(torch.bfloat16)
    ow = torch.empty_like(w)
    mw = torch.empty((16384, 1), dtype=torch.int32, device="cuda")
    add("c3_per_row_e4m3_16384x4096", lambda: run.fake_quantize(w, ow, mw, 1, 4096, 0.0, 2, 1), w.numel() * 4 + 16384 * 4, w.numel())
    add("c3_per_row_e5m2_16384x4096", lambda: run.fake_quantize(w, ow, mw, 1, 4096, 0.0, 3, 1), w.numel() * 4 + 16384 * 4, w.numel())
    st3 = run.scaling_state(16384, 4096, 1, 4096, True)
    add("c3_per_row_e4m3_16384x4096_channel_op_ss3", lambda: run.block_scaling(w, ow, st3, 1, 4096, 0.045, 3), w.numel() * 4, w.numel())   # block-local scale: one pass
    del w, ow
    # C4: MoR 128x128 on the 16384x14336 mixture
    x4 = gen_c4_gpu(torch, 16384, 14336)
    o4 = torch.empty_like(x4)
    m4 = torch.empty((128, 112), dtype=torch.int32, device="cuda")
    add("c4_mor_128x128_16384x14336_mixture", lambda: run.fake_quantize(x4, o4, m4, 128, 128, 1e-15, 1, 1), x4.numel() * 4 + m4.numel() * 4, x4.numel())
    torch.cuda.synchronize()
    hist = torch.bincount(m4.flatten(), minlength=13).tolist()
    res["c4_mor_128x128_16384x14336_mixture"]["meta_histogram"] = {str(i): h for i, h in enumerate(hist) if h}
    mor_tile_codes(torch, cabi, run, add, x4, o4, "16384x14336_mixture")
    del x4, o4
    res["flavour_differences"] = flavour_differences(torch, run, cabi)
    res["c5_llama3_8b_layer"] = c5_sweep(torch, run, max(3, K // 4), 2)
    res["mx_wire_format_8192x8192"] = wire_format(torch, run, K, W)
    # launch overhead: a 1x32 tensor
    xs = torch.randn(1, 32, device="cuda").to(torch.bfloat16)
    os_ = torch.empty_like(xs)
    ms_ = torch.empty((1, 1), dtype=torch.int32, device="cuda")
    ms, wall = time_launches(torch, lambda: run.fake_quantize(xs, os_, ms_, 1, 32, 0.0, 2, 2), 200, 20)
    res["tiny_1x32"] = {"us_per_call_events": round(ms * 1e3, 2), "us_per_call_wall": round(wall * 1e3, 2)}
    # 100 such calls captured in a HIP graph (the C ABI allocates nothing and clears with kernels): per call on replay
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        run.fake_quantize(xs, os_, ms_, 1, 32, 0.0, 2, 2)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(100):
            run.fake_quantize(xs, os_, ms_, 1, 32, 0.0, 2, 2)
    ms, wall = time_launches(torch, graph.replay, 20, 3)
    res["tiny_1x32"]["graph_replay_us_per_call"] = round(ms * 1e3 / 100, 2)
    # 100 separate 1x32 tensors through the batch entry: two launches for all of them
    from mor_amd.batch import BatchPlan
    for mode, key in ((2, "batch_100_tensors_e4m3_us_per_tensor"), (1, "batch_100_tensors_mor_us_per_tensor")):
        pool_x = torch.randn(100, 32, device="cuda").to(torch.bfloat16)
        pool_o = torch.empty_like(pool_x)
        pool_m = torch.empty((100, 1), dtype=torch.int32, device="cuda")
        plan = BatchPlan([pool_x[i:i + 1] for i in range(100)], [pool_o[i:i + 1] for i in range(100)],
                         [pool_m[i:i + 1] for i in range(100)], [(1, 32)] * 100, 1e-3, mode, 2)
        ms, wall = time_launches(torch, plan.run, 200, 20)
        res["tiny_1x32"][key] = round(ms * 1e3 / 100, 3)
        res["tiny_1x32"][key.replace("_us_", "_wall_us_")] = round(wall * 1e3 / 100, 3)
    # the seven weight matrices of a Llama-3-8B layer (q, k, v, o, gate, up, down: 872 MB of traffic) in one call: their
    # 128 x 128 tiles run as grids of one tile kernel (tensors of one streaming class share a launch)
    wshapes = [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096), (4096, 14336)]
    gw = torch.Generator(device="cuda").manual_seed(1005)
    wx = [(torch.randn(r, c, device="cuda", generator=gw) * 0.02).to(torch.bfloat16) for r, c in wshapes]
    wo = [torch.empty_like(t) for t in wx]
    wm = [torch.empty((r // 128, c // 128), dtype=torch.int32, device="cuda") for r, c in wshapes]
    wbytes = sum(t.numel() for t in wx) * 4
    res["llama3_8b_weights_one_call"] = {"bytes": wbytes}
    for mode, key in ((1, "mor_128x128"), (2, "block_e4m3_128x128")):
        plan = BatchPlan(wx, wo, wm, [(128, 128)] * 7, 1e-15, mode, 1)
        ms, wall = time_launches(torch, plan.run, 60, 200)
        one = 0.0
        for t, o, m in zip(wx, wo, wm):
            ms1, _ = time_launches(torch, lambda: run.fake_quantize(t, o, m, 128, 128, 1e-15, mode, 1), 100, 300)
            one += ms1
        res["llama3_8b_weights_one_call"][key] = {"ms": round(ms, 5), "GBps": round(wbytes / (ms * 1e-3) / 1e9, 1), "frac": round(wbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                                  "seven_calls_ms": round(one, 5)}
    del wx, wo
    # the same call through the operator layer a user of the reference calls (allocations of out and meta included)
    import mor
    xg = xs.clone().requires_grad_(True)
    for key, t in (("mor_ops_us_per_call", xs), ("mor_ops_requires_grad_us_per_call", xg)):
        ms, wall = time_launches(torch, lambda: mor.ops.fake_quantize(t, 1, 32, 1, 32, 0.0, 2, 2), 500, 50)
        res["tiny_1x32"][key] = round(wall * 1e3, 2)
    return res


def mor_tile_codes(torch, cabi, run, add, x, out, label):
    """MoR per 128 x 128 tile with the codes as the result (tag + fp32 scale + payload) and the decode back to bf16.
    Bytes: the bf16 tensor on one side, on the other what the tiles' formats take (1 B/element for E4M3 / E5M2, 0.75 for
    E2M3, 2 for BF16) plus 8 bytes of tag and scale per tile."""
    from mor_amd.wire import TILE_PAYLOAD_BYTES, TILE_STORED_BF16
    rows, cols = x.shape
    gy, gx = rows // 128, cols // 128
    payload = torch.empty((gy, gx, TILE_PAYLOAD_BYTES), dtype=torch.uint8, device="cuda")
    tags = torch.empty((gy, gx), dtype=torch.int32, device="cuda")
    scales = torch.empty((gy, gx), dtype=torch.float32, device="cuda")
    L, st = run.L, run.stream
    enc = lambda: cabi.check(L.mor_mor_quantize(x.data_ptr(), payload.data_ptr(), tags.data_ptr(), scales.data_ptr(), rows, cols, 1e-15, 1, st()))
    dec = lambda: cabi.check(L.mor_mor_dequantize(payload.data_ptr(), tags.data_ptr(), scales.data_ptr(), out.data_ptr(), rows, cols, st()))
    enc()
    torch.cuda.synchronize()
    t = tags.flatten()
    wide = ((t & TILE_STORED_BF16) != 0) | (t == 3)
    code_bytes = int(wide.sum()) * 32768 + int(((t == 4) & ~wide).sum()) * 12288 + int((~wide & (t != 4)).sum()) * 16384
    n = x.numel()
    add("mor_tile_codes_quantize_" + label, enc, 2 * n + code_bytes + 8 * t.numel(), n)
    add("mor_tile_codes_dequantize_" + label, dec, 2 * n + code_bytes + 8 * t.numel(), n)
    # the codes of the transposed tensor from the codes (tile by tile through LDS): the codes are read once and written once
    payload_t, tags_t, scales_t = torch.empty_like(payload).view(gx, gy, TILE_PAYLOAD_BYTES), torch.empty((gx, gy), dtype=torch.int32, device="cuda"), torch.empty((gx, gy), dtype=torch.float32, device="cuda")
    tr = lambda: cabi.check(L.mor_mor_transpose(payload.data_ptr(), tags.data_ptr(), scales.data_ptr(), payload_t.data_ptr(), tags_t.data_ptr(),
                                                scales_t.data_ptr(), gy, gx, st()))
    add("mor_tile_codes_transpose_" + label, tr, 2 * code_bytes + 16 * t.numel(), n)
    # both in one call (two launches)
    both = lambda: cabi.check(L.mor_mor_quantize_dual(x.data_ptr(), payload.data_ptr(), tags.data_ptr(), scales.data_ptr(), payload_t.data_ptr(),
                                                      tags_t.data_ptr(), scales_t.data_ptr(), rows, cols, 1e-15, 1, st()))
    add("mor_tile_codes_quantize_dual_" + label, both, 2 * n + 2 * code_bytes + 16 * t.numel(), n)


def flavour_differences(torch, run, cabi):
    """Per configuration, the number of elements on which the two flavours of the library differ: what the reference's
    CUDA kernel returns (the default: round-half-up bf16 store, exponent-field power-of-two scaling, +0 from the
    software cast) against what its torch emulation returns (nearest-even store, true zeros, signed zeros)."""
    EMU = cabi.FLAG_TORCH_EMULATION
    res = {}

    def count(name, x, call):
        a, b = torch.empty_like(x), torch.empty_like(x)
        call(a, 0)
        call(b, EMU)
        torch.cuda.synchronize()
        d = a.view(torch.int16) != b.view(torch.int16)
        res[name] = {"elements": x.numel(), "differ": int(d.sum().item()),
                     "differ_ignoring_sign_of_zero": int((d & ((a != 0) | (b != 0))).sum().item())}

    g = torch.Generator(device="cuda").manual_seed(1001)
    x1 = torch.randn(4096, 4096, device="cuda", generator=g).to(torch.bfloat16)
    m = torch.empty(4096 * 4096 // 32, dtype=torch.int32, device="cuda")
    scale = float(448.0 / x1.float().abs().max().item())
    count("c1_per_tensor_e4m3_4096x4096", x1, lambda o, f: run.fake_quantize(x1, o, m, 128, 128, scale, 4, 1, f))
    x2 = gen_c2_gpu(torch, 4096, 8192)
    m2 = torch.empty(x2.numel() // 32, dtype=torch.int32, device="cuda")
    count("c2_mx_e4m3_half_tensor", x2, lambda o, f: run.fake_quantize(x2, o, m2, 1, 32, 0.0, 2, 2, f))
    count("c2_mx_e5m2_half_tensor", x2, lambda o, f: run.fake_quantize(x2, o, m2, 1, 32, 0.0, 3, 2, f))
    count("c2_mx_e2m3_half_tensor", x2, lambda o, f: run.block_format(x2, o, 1, 32, cabi.FMT_E2M3, 2, f))
    g = torch.Generator(device="cuda").manual_seed(1003)
    w = torch.randn(8192, 4096, device="cuda", generator=g) * 0.02
    w[torch.randperm(8192, device="cuda", generator=g)[:82]] *= 100
    w[7] = 0
    w = w.to(torch.bfloat16)
    count("c3_per_row_e4m3_half_tensor", w, lambda o, f: run.fake_quantize(w, o, m, 1, 4096, 0.0, 2, 1, f))
    count("c3_per_row_e5m2_half_tensor", w, lambda o, f: run.fake_quantize(w, o, m, 1, 4096, 0.0, 3, 1, f))
    x4 = gen_c4_gpu(torch, 4096, 14336)
    count("c4_mor_128x128_quarter_tensor", x4, lambda o, f: run.fake_quantize(x4, o, m, 128, 128, 1e-15, 1, 1, f))
    return res


def wire_format(torch, run, K, W):
    """The MX wire format on the benchmark tensor: codes + E8M0 scale bytes (2 B read + 1 or 0.75 B written per element
    + 1 scale byte per block), both orientations from one read, and the decode."""
    L = run.L
    rows = cols = 8192
    x = gen_c2_gpu(torch, rows, cols)
    n = rows * cols
    out = {}
    for fmt, name, bits in ((run.cabi.FMT_E4M3, "e4m3", 8), (run.cabi.FMT_E5M2, "e5m2", 8), (run.cabi.FMT_E2M3, "e2m3", 6)):
        pb = n * bits // 8
        p = torch.empty(pb, dtype=torch.uint8, device="cuda")
        s = torch.empty(n // 32, dtype=torch.uint8, device="cuda")
        cp, cs, o = torch.empty_like(p), torch.empty_like(s), torch.empty_like(x)
        for key, fn, nbytes in (
            ("quantize", lambda: run.cabi.check(L.mor_mx_quantize(x.data_ptr(), p.data_ptr(), s.data_ptr(), rows, cols, fmt, run.stream())), 2 * n + pb + n // 32),
            ("quantize_dual", lambda: run.cabi.check(L.mor_mx_quantize_dual(x.data_ptr(), p.data_ptr(), s.data_ptr(), cp.data_ptr(), cs.data_ptr(), rows, cols, fmt, run.stream())), 2 * n + 2 * (pb + n // 32)),
            ("dequantize", lambda: run.cabi.check(L.mor_mx_dequantize(p.data_ptr(), s.data_ptr(), o.data_ptr(), rows, cols, fmt, run.stream())), 2 * n + pb + n // 32),
        ):
            ms = time_launches(torch, fn, K, W)[0]
            out[f"{key}_{name}"] = {"us": round(ms * 1e3, 1), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                                    "frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    # fake quantization of the tensor and of its transpose from one read (2 B read + 4 B written per element + meta)
    o, ot = torch.empty_like(x), torch.empty_like(x)
    m, mt = (torch.empty(n // 32, dtype=torch.int32, device="cuda") for _ in range(2))
    ms = time_launches(torch, lambda: run.cabi.check(L.mor_fake_quantize_dual(x.data_ptr(), o.data_ptr(), m.data_ptr(), ot.data_ptr(),
                                                                              mt.data_ptr(), rows, cols, 2, 2, run.stream())), K, W)[0]
    nbytes = 6 * n + 2 * (n // 32) * 4
    out["fake_quantize_dual_e4m3"] = {"us": round(ms * 1e3, 1), "GBps": round(nbytes / (ms * 1e-3) / 1e9, 1),
                                      "frac": round(nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    return out


def c5_sweep(torch, run, K, W):
    """Every tensor one Llama-3-8B layer quantizes in a forward + backward pass at 16384 tokens: activations and
    output gradients N(0,1), weights N(0,0.02).  Three families: MoR 128x128, block E4M3 128x128, and per-channel
    (row-wise for fprop / dgrad, column-wise blocks N x 1 through the channel-scaling op for wgrad).  Per family:
    total algorithmic bytes / total kernel time; per shape: microseconds and GB/s.  Plus the ragged 4097 x 4095."""
    T, D, KV, F = 16384, 4096, 1024, 14336
    acts = [("x_qkv", T, D), ("attn_out", T, D), ("x_mlp", T, D), ("h_down", T, F)]
    weights = [("wq", D, D), ("wk", KV, D), ("wv", KV, D), ("wo", D, D), ("w_gate", F, D), ("w_up", F, D), ("w_down", D, F)]
    grads = [("dy_q", T, D), ("dy_o", T, D), ("dy_down", T, D), ("dy_k", T, KV), ("dy_v", T, KV), ("dy_gate", T, F), ("dy_up", T, F)]
    g = torch.Generator(device="cuda").manual_seed(1005)
    big = torch.randn(T * F, device="cuda", generator=g).to(torch.bfloat16)
    small = (torch.randn(F * D, device="cuda", generator=g) * 0.02).to(torch.bfloat16)
    obuf = torch.empty_like(big)
    mbuf = torch.empty(T * F // 32, dtype=torch.int32, device="cuda")
    cache = {}

    def timed(key, fn):
        # every shape is timed over about 10 ms of back-to-back launches: a burst of a few hundred microseconds ends
        # before the clocks have left their idle state, and a millisecond is still noisy
        if key not in cache:
            ms = time_launches(torch, fn, K, W)[0]
            if ms * K < 10.0:
                ms = time_launches(torch, fn, min(1000, int(10.0 / ms) + 1), W)[0]
            cache[key] = ms
        return cache[key]

    def view(src, r, c):
        return src[: r * c].view(r, c)

    fam = {}
    # the buffers are fresh: the first tens of milliseconds on them run slower (first touch), so they are not timed
    xw, ow = view(big, T, D), view(obuf, T, D)
    for _ in range(300):
        run.fake_quantize(xw, ow, mbuf, 128, 128, 1e-15, 1, 1)
    torch.cuda.synchronize()

    def family(name, entries):
        tot_b = tot_ms = 0.0
        shapes = {}
        for tname, r, c, src, kind in entries:
            x, o = view(src, r, c), view(obuf, r, c)
            tag = "w" if src is small else "a"
            if kind == "mor":
                ms = timed((tag, r, c, kind), lambda: run.fake_quantize(x, o, mbuf, 128, 128, 1e-15, 1, 1))
                nb = r * c * 4 + (r // 128) * (c // 128) * 4
            elif kind == "block":
                ms = timed((tag, r, c, kind), lambda: run.fake_quantize(x, o, mbuf, 128, 128, 0.0, 2, 1))
                nb = r * c * 4 + (r // 128) * (c // 128) * 4
            elif kind == "row":
                ms = timed((tag, r, c, kind), lambda: run.fake_quantize(x, o, mbuf, 1, c, 0.0, 2, 1))
                nb = r * c * 4 + r * 4
            else:                                   # column blocks r x 1: channel-scaling op, fp32 scale per column
                st = run.scaling_state(r, c, r, 1, True)
                ms = timed((tag, r, c, kind), lambda: run.block_scaling(x, o, st, r, 1, 0.045, 3))
                nb = r * c * 6
            tot_b += nb
            tot_ms += ms
            shapes[f"{r}x{c}_{tag}_{kind}"] = {"us": round(ms * 1e3, 1), "GBps": round(nb / (ms * 1e-3) / 1e9, 1)}
        fam[name] = {"launches": len(entries), "total_ms": round(tot_ms, 4), "total_GB": round(tot_b / 1e9, 3),
                     "GBps": round(tot_b / (tot_ms * 1e-3) / 1e9, 1), "frac": round(tot_b / (tot_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "shapes": shapes}

    every = [(n, r, c, big) for n, r, c in acts + grads] + [(n, r, c, small) for n, r, c in weights]
    family("mor_128x128", [(n, r, c, s, "mor") for n, r, c, s in every])
    family("block_e4m3_128x128", [(n, r, c, s, "block") for n, r, c, s in every])
    family("per_channel_rows_and_columns", [(n, r, c, s, "row") for n, r, c, s in every]
           + [(n, r, c, big, "col") for n, r, c in acts + grads])
    # ragged, odd column count (scalar kernel): a shape the reference rejects
    xr, orr = view(big, 4097, 4095), view(obuf, 4097, 4095)
    ms = time_launches(torch, lambda: run.fake_quantize(xr, orr, mbuf, 128, 128, 1e-15, 1, 1), K, W)[0]
    fam["ragged_4097x4095_mor_128x128"] = {"us": round(ms * 1e3, 1), "GBps": round(4097 * 4095 * 4 / (ms * 1e-3) / 1e9, 1)}
    return fam


def cpu_baseline(torch, x_gpu, x_mor_gpu):
    """The CPU oracle (a port of the reference arithmetic, OpenMP over blocks, all host threads) on bounded samples:
    the benchmark step (`value`) and one row per configuration (`per_config`), each about two seconds of CPU work; plus
    a vectorised restatement of the reference's torch emulation (its own CPU path, test/test_fake_quantize.py:33-143,
    432-436) where that exists for the configuration."""
    from oracle import mor_oracle as O
    import numpy as np
    sys.path.insert(0, os.path.join(ROOT, "tests"))          # the CPU leg restates the reference's torch emulation: test infrastructure
    import torch_emulation as E
    O.lib()
    torch.set_num_threads(os.cpu_count() or 1)

    def bits(t):
        return t.contiguous().cpu().view(torch.int16).numpy().view(np.uint16).copy()

    def timed(fn, budget_s, max_reps=200):
        fn()                                           # warm-up (page faults, thread pool)
        reps, t_total, t_start = 0, 0.0, time.perf_counter()
        while True:
            t0 = time.perf_counter()
            fn()
            t_total += time.perf_counter() - t0
            reps += 1
            if time.perf_counter() - t_start > budget_s or reps >= max_reps:
                return t_total / reps, reps

    rows = 2048
    a = bits(x_gpu[:rows])
    am = bits(x_mor_gpu[:rows])
    n = a.size
    step_bytes = 4 * n * 4 + 2 * (n // 32) * 4 + (n // 16384) * 4

    def step():
        O.fake_quantize(a, 1, 32, 0.0, 2, 2)
        O.fake_quantize(a, 1, 32, 0.0, 3, 2)
        O.block_format(a, 1, 32, O.E2M3, 2)
        O.fake_quantize(am, 128, 128, 1e-15, 1, 1)

    sec, reps = timed(step, 6.0)
    res = {"value": round(step_bytes / sec / 1e9, 3), "unit": "GB/s", "cores": O.num_threads(), "kind": "port",
           "sample": f"first {rows} rows of the two benchmark tensors ({n} elements each): MX E4M3 + E5M2 + E2M3 and MoR 128x128, "
                     f"{reps} repetitions, C oracle with OpenMP over blocks"}
    per = {}

    def row(name, nbytes, what, oracle_fn, emu_fn=None, budget=2.0):
        sec, reps = timed(oracle_fn, budget)
        per[name] = {"oracle_GBps": round(nbytes / sec / 1e9, 3), "elements_per_s": round(nbytes / 4 / sec, 0), "sample": what, "repetitions": reps}
        if emu_fn is not None:
            try:
                sec, reps = timed(emu_fn, budget, 20)
                per[name]["torch_emulation_GBps"] = round(nbytes / sec / 1e9, 3)
            except Exception as e:                                   # the emulation is a courtesy figure, never a failure
                per[name]["torch_emulation_error"] = repr(e)

    # C1: the reference's own CPU-runnable case, at full size: per-tensor E4M3 on 4096 x 4096 N(0,1)
    g = torch.Generator().manual_seed(1001)
    t1 = torch.randn(4096, 4096, generator=g).to(torch.bfloat16)
    a1 = bits(t1)
    amax1 = t1.float().abs().max().item()
    s1 = float(np.float32(448.0) / np.float32(amax1))
    row("c1_per_tensor_e4m3_4096x4096", a1.size * 4, "the whole tensor, scale 448 / amax",
        lambda: O.fake_quantize(a1, 128, 128, s1, 4, 1),
        lambda: E.quant_dequant_scaled(t1.float(), "e4m3", amax1).to(torch.bfloat16))
    row("c2_mx_e4m3_8192x8192", n * 4, f"first {rows} rows", lambda: O.fake_quantize(a, 1, 32, 0.0, 2, 2),
        lambda: E.block_format_fast(a, 1, 32, "e4m3", e8=True))
    a3 = a.reshape(rows * 2, 4096)
    row("c3_per_row_e4m3_16384x4096", a3.size * 4, f"{a3.shape[0]} rows of 4096 elements", lambda: O.fake_quantize(a3, 1, 4096, 0.0, 2, 1),
        lambda: E.block_format_fast(a3, 1, 4096, "e4m3"))
    a4 = bits(gen_c4_gpu(torch, 1024, 14336))
    row("c4_mor_128x128_16384x14336", a4.size * 4, "1024 rows of the tile mixture (896 tiles)", lambda: O.fake_quantize(a4, 128, 128, 1e-15, 1, 1))
    res["per_config"] = per
    try:
        with open("/proc/cpuinfo") as f:
            res["cpu_model"] = next((l.split(":", 1)[1].strip() for l in f if l.startswith("model name")), "unknown")
    except OSError:
        pass
    return res


if __name__ == "__main__":
    main()
