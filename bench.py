#!/usr/bin/env python3
"""Benchmark of the 4-bit group-quantization path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only decompress|compress|gemv|kn|knp|gemm|stack|all]

One "step" is one standalone int4 -> fp16 decompress of the 4096 x 16384 weight (benchmark
configuration 2: group 64, ~N(0, 0.02) with 0.1 % outliers at +-8 sigma, packed by the
device-side packer that the tests hold bit-identical to the numpy packer).  Inputs are resident in
HBM before the timed region; buffer sets are rotated so that the working set (4 x 172 MB) does not
fit the 256 MB last-level cache.  The fused GEMV / GEMM / layer-stack measurements of the other
configurations are summarised in the same JSON line under "extra" (one short record per shape);
every figure of the run goes to the detail file (--detail) and to stderr.

The LAST line on stdout is the one JSON line (under 4 KB); progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "popxl-addons_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16, published
GROUP = 64
# HBM bytes per decompress launch, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE: the summary
# of those runs holds one machine-readable line with the figure and the commit it was taken at
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "decompress_kernel_4096x16384.md")


def measured_traffic():
    """(bytes per launch, commit) from the committed profile summary, or (None, None)."""
    import re

    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None, None
    m = re.search(r"traffic_bytes_per_launch\s*=\s*(\d+)\s+at commit\s+([0-9a-f]{7,40})", text)
    return (int(m.group(1)), m.group(2)) if m else (None, None)


def hbm_roofline(kernel, nbytes, ms, **more):
    gbs = nbytes / ms / 1e6
    return dict({"kernel": kernel, "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                 "frac": round(gbs / HBM_PEAK_GBS, 4), "algorithmic_bytes_per_launch": nbytes}, **more)


def mfma_roofline(kernel, flops, ms, **more):
    tf = flops / ms / 1e9
    return dict({"kernel": kernel, "bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                 "frac": round(tf / MFMA_F16_PEAK_TFLOPS, 4), "algorithmic_flops_per_launch": flops}, **more)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def stream_handle():
    import torch

    return torch.cuda.current_stream().cuda_stream


def time_launches(fn, steps, warmup):
    """Average milliseconds of fn(i) over `steps` back-to-back launches on the current stream (HIP events)."""
    import torch

    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        fn(i)
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def run_until_steady(fn, seconds=0.03):
    """Untimed launches of fn(i) for `seconds`.  The first launches after a pause (here: after the
    operands were made) run slower than the steady state -- the fused GEMV on 16384x4096 at batch 8:
    14.0, 13.4, 13.0, 12.0 us over the first four blocks of 200 launches, 11.8 us from then on; the
    packer on 4096x16384: 31.7, 32.8, 31.7, 31.4, 30.9, 30.8 us over the first six blocks of 100,
    30.3 - 30.5 us from the eighth on.  Used by the benchmarks under `extra`; the headline decompress
    figure is timed after exactly --warmup launches."""
    import torch

    t0, i0 = time.time(), 0
    while time.time() - t0 < seconds:
        for i in range(100):
            fn(i0 + i)
        i0 += 100
        torch.cuda.synchronize()


def make_weight(n_rows, n_cols, seed, outliers, device):
    """fp16 weight ~N(0, 0.02) (+ 0.1 % outliers at +-0.16), generated on the device from a seed."""
    import torch

    g = torch.Generator(device=device)
    g.manual_seed(seed)
    w = torch.randn((n_rows, n_cols), generator=g, device=device, dtype=torch.float32) * 0.02
    if outliers:
        u = torch.rand((n_rows, n_cols), generator=g, device=device)
        w = torch.where(u < 5e-4, torch.full_like(w, 0.16), w)
        w = torch.where(u > 1 - 5e-4, torch.full_like(w, -0.16), w)
    return w.to(torch.float16)


def pack_weight(w):
    from popxl_addons.ops.group_quantize_decompress import group_quantize_compress

    return group_quantize_compress(w, GROUP)


# --------------------------------------------------------------------------------- decompress


def bench_decompress(hip, device, steps, warmup, n_sets=4, rows=4096, cols=16384):
    import torch

    sets = []
    for s in range(n_sets):
        packed, scale, bias = pack_weight(make_weight(rows, cols, 100 + s, True, device))
        out = torch.empty((rows, cols), dtype=torch.float16, device=device)
        sets.append((packed, scale, bias, out))
    torch.cuda.synchronize()
    n_groups, n_ids = cols // GROUP, GROUP // 4
    stream = stream_handle()

    def step(i):
        p, s, b, o = sets[i % n_sets]
        hip.call("gq_decompress_f16", p.data_ptr(), s.data_ptr(), b.data_ptr(), o.data_ptr(), rows, n_groups, n_ids, stream)

    ms = time_launches(step, steps, warmup)
    # algorithmic bytes per launch: 0.5 B codes + 4/gs B scale/bias read, 2 B written per element
    bytes_per_launch = rows * cols * (0.5 + 4.0 / GROUP + 2.0)
    return {"ms": ms, "bytes": bytes_per_launch, "gbs": bytes_per_launch / ms / 1e6, "sets": sets}


def bench_compress(hip, device, steps, warmup, n_sets=4, rows=4096, cols=16384, f32=False):
    """Device-side packer on the configuration-2 weight: reads 2 B (4 B for float32 input), writes
    0.5 + 4/gs B per element."""
    import torch

    sets = []
    for s in range(n_sets):
        w = make_weight(rows, cols, 100 + s, True, device)
        if f32:
            w = w.float()
        n_groups = cols // GROUP
        sets.append((w, torch.empty((rows, n_groups, GROUP // 4), dtype=torch.uint16, device=device),
                     torch.empty((rows, n_groups, 1), dtype=torch.float16, device=device),
                     torch.empty((rows, n_groups, 1), dtype=torch.float16, device=device)))
    flag = torch.zeros(1, dtype=torch.int32, device=device)
    stream = stream_handle()

    def step(i):
        w, p, s, b = sets[i % n_sets]
        hip.call("gq_compress_f32" if f32 else "gq_compress_f16", w.data_ptr(), p.data_ptr(), s.data_ptr(), b.data_ptr(),
                 flag.data_ptr(), rows, cols // GROUP, GROUP, stream)

    run_until_steady(step)
    ms = time_launches(step, steps, warmup)
    nbytes = rows * cols * ((4.0 if f32 else 2.0) + 0.5 + 4.0 / GROUP)
    return {"rows": rows, "cols": cols, "input": "float32" if f32 else "float16", "us": ms * 1e3, "bytes": nbytes,
            "gbs": nbytes / ms / 1e6, "hbm_frac": nbytes / ms / 1e6 / HBM_PEAK_GBS,
            "roofline": hbm_roofline("compress_f32_kernel" if f32 else "compress_kernel", nbytes, ms)}


def _blas_threads():
    try:
        from threadpoolctl import threadpool_info

        return max([p.get("num_threads", 1) for p in threadpool_info() if p.get("user_api") == "blas"] or [1])
    except Exception:  # noqa: BLE001 (a reporting aid only)
        return None


def _best_of(fn, repeats=3):
    best, out = 1e30, None
    for _ in range(repeats):
        t0 = time.perf_counter()
        out = fn()
        best = min(best, time.perf_counter() - t0)
    return best, out


def cpu_baseline_decompress(sets, rows_sample=4096):
    """The numpy restatement of the reference's decompress (oracle/), timed on the host cores on one
    full 4096 x 16384 weight, best of 3.  numpy's elementwise passes run on one thread."""
    from oracle import gq_oracle

    p, s, b, _ = sets[0]
    p, s, b = (a[:rows_sample].cpu().numpy() for a in (p, s, b))
    best, out = _best_of(lambda: gq_oracle.np_decompress(p, s, b))
    n_bytes = p.nbytes + s.nbytes + b.nbytes + out.nbytes
    return {
        "value": n_bytes / best / 1e9,
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "sample": f"numpy decompress of one {p.shape[0]}x{out.shape[1]} weight (group 64), best of 3, {best:.3f} s; "
        f"host has {os.cpu_count()} cpus, {len(os.sched_getaffinity(0))} usable, numpy elementwise = 1 thread",
    }, out


def cpu_baseline_legs():
    """The other CPU legs: configuration 1 decompress, and decompress -> float32 matmul (what the
    reference's layer computes on the host, tests/integration/layers/test_linear_gq.py:18-30) for
    configuration 3 (both shapes, batch 1) and configuration 4 (batch 128).  Same units as the
    GPU rows they stand beside; seeded numpy inputs, the numpy packer."""
    import numpy as np
    from oracle import gq_oracle
    from popxl_addons.ops.group_quantize_decompress import group_quantize_compress_numpy

    rng = np.random.default_rng(1)
    legs = []
    w = rng.normal(0, 0.02, (1024, 1024)).astype(np.float16)
    packed, scale, bias = group_quantize_compress_numpy(w, GROUP)
    best, out = _best_of(lambda: gq_oracle.np_decompress(packed, scale, bias))
    nbytes = packed.nbytes + scale.nbytes + bias.nbytes + out.nbytes
    legs.append({"workload": "config 1: numpy decompress 1024x1024", "seconds": best, "value": nbytes / best / 1e9,
                 "unit": "GB/s (read + written)", "cores": 1})
    blas = _blas_threads()
    for m_rows, n_out, k_in, name in ((1, 4096, 4096, "config 3"), (1, 16384, 4096, "config 3"), (128, 16384, 4096, "config 4")):
        w = rng.normal(0, 0.02, (n_out, k_in)).astype(np.float16)
        packed, scale, bias = group_quantize_compress_numpy(w, GROUP)
        x = rng.normal(0, 1, (m_rows, k_in)).astype(np.float16)
        best, _ = _best_of(lambda: gq_oracle.np_linear(x, gq_oracle.np_decompress(packed, scale, bias)), repeats=2)
        w_bytes = n_out * k_in * (0.5 + 4.0 / GROUP)
        legs.append({"workload": f"{name}: numpy decompress -> float32 matmul, m={m_rows} [{n_out}x{k_in}]", "seconds": best,
                     "value": w_bytes / best / 1e9, "unit": "GB/s (packed weight bytes)",
                     "tflops": 2.0 * m_rows * n_out * k_in / best / 1e12, "cores": f"decompress 1, BLAS {blas}"})
    return legs


# -------------------------------------------------------------------------------------- fused


def sets_beyond_cache(n_out, k_in):
    """Distinct weights to rotate over so that their packed bytes (> 600 MB) cannot stay in the
    256 MB last-level cache from one launch to the next."""
    return max(2, int(600e6 // (n_out * k_in * (0.5 + 4.0 / GROUP))) + 1)


def one_shot_kernel_name(m_rows, n_out, k_in):
    """The kernel that a single fused GEMV of this shape runs on (weights grouped along the input features, group 64,
    k_in % 512 == 0, aligned operands): the library's routing, restated for the labels of the rows."""
    if m_rows <= 2:
        return "gemv_sums_kernel"
    if m_rows <= 8 and k_in <= 4096 and ((n_out + 15) // 16 + 7) // 8 >= 208:
        return "gemv_rows_kernel"
    if m_rows <= 4 and n_out * k_in >= (72 << 20) and k_in < 8192:
        return "gemv_stream_kernel as a sequence of one"
    return "gemv_mfma_kernel"


def bench_linear(hip, device, entry, m_rows, n_out, k_in, steps, warmup, n_sets, kernel):
    """One fused dequant matmul shape; weights rotated over n_sets distinct copies.  `entry` is
    gq_gemv_f16 / gq_gemm_f16 (weight [n_out, k_in], groups along k_in) or gq_linear_kn_act_f16
    (weight [k_in, n_out], groups along n_out: the default layout of LinearGQ)."""
    import torch

    knp = entry == "gq_linear_knp_act_f16"  # (the same layout, read from its derived copy: the kn streaming layout)
    nkp = entry == "gq_linear_p_act_f16"  # (groups along k_in: the variables AND their derived copy in the streaming layout)
    kn = entry == "gq_linear_kn_act_f16" or knp
    sets = []
    for s in range(n_sets):
        w = make_weight(k_in, n_out, 200 + s, False, device) if kn else make_weight(n_out, k_in, 200 + s, False, device)
        sets.append((hip.prepack_gemv_kn(*pack_weight(w)),) if knp else pack_weight(w))
        if nkp:
            sets[-1] = sets[-1] + (hip.prepack_gemv(*sets[-1]),)
    g = torch.Generator(device=device)
    g.manual_seed(7)
    x = torch.randn((m_rows, k_in), generator=g, device=device, dtype=torch.float32).to(torch.float16)
    y = torch.empty((m_rows, n_out), dtype=torch.float16, device=device)
    stream = stream_handle()
    with_ws = entry == "gq_linear_act_ws_f16"  # (the layer's entry for the [n_out, k_in] layout: K may be divided over workgroups)
    ws_bytes = (0 if knp else hip.load().gq_linear_kn_workspace_bytes(m_rows, n_out, k_in, GROUP) if kn else
                hip.load().gq_gemm_workspace_bytes(m_rows, n_out, k_in, GROUP) if with_ws else 0)
    ws = torch.zeros(max(ws_bytes, 16), dtype=torch.uint8, device=device)

    def step(i):
        if knp:
            hip.call(entry, x.data_ptr(), m_rows, sets[i % n_sets][0].blob.data_ptr(), 0, y.data_ptr(), n_out, k_in, GROUP, 0, stream)
            return
        if nkp:
            p, s, b, copy = sets[i % n_sets]
            hip.call(entry, x.data_ptr(), m_rows, p.data_ptr(), s.data_ptr(), b.data_ptr(), copy.blob.data_ptr(), 0, y.data_ptr(), n_out,
                     k_in, GROUP, 0, 0, 0, stream)
            return
        p, s, b = sets[i % n_sets]
        if kn:
            hip.call(entry, x.data_ptr(), m_rows, p.data_ptr(), s.data_ptr(), b.data_ptr(), 0, y.data_ptr(), n_out, k_in, GROUP,
                     0, ws.data_ptr(), ws.numel(), stream)
        elif with_ws:
            hip.call(entry, x.data_ptr(), m_rows, p.data_ptr(), s.data_ptr(), b.data_ptr(), 0, y.data_ptr(), n_out, k_in, GROUP,
                     0, ws.data_ptr(), ws.numel(), stream)
        else:
            hip.call(entry, x.data_ptr(), m_rows, p.data_ptr(), s.data_ptr(), b.data_ptr(), 0, y.data_ptr(), n_out, k_in, GROUP, stream)

    run_until_steady(step)
    ms = time_launches(step, steps, warmup)
    w_bytes = n_out * k_in * (0.5 + 4.0 / GROUP)
    flops = 2.0 * m_rows * n_out * k_in
    r = {
        "m": m_rows, "n": n_out, "k": k_in, "layout": "[k_in, n_out]" if kn else "[n_out, k_in]", "n_sets": n_sets, "us": ms * 1e3,
        "weight_gbs": w_bytes / ms / 1e6, "hbm_frac": w_bytes / ms / 1e6 / HBM_PEAK_GBS,
        "tflops": flops / ms / 1e9, "mfma_frac": flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS,
    }
    # decode batches are bound by the packed weight bytes, prefill batches by the fp16 MFMA rate
    r["roofline"] = hbm_roofline(kernel, w_bytes, ms) if m_rows <= 16 else mfma_roofline(kernel, flops, ms)
    return r


FLOW_KERNEL_MODES = ("sequence_decoder_data_flow_streaming_layout", "sequence_decoder_data_flow_joint_output_streaming_layout",
                     "sequence_decoder_data_flow_two_entries_streaming_layout",
                     "sequence_no_waits_streaming_layout")


def bench_stack(hip, device, m_rows, passes, warmup, n_layers=28, hidden=4096, ffn=16384, modes=None, oracle=None):
    """Benchmark configuration 5: 28 layers x {4 x [4096x4096], [16384x4096], [4096x16384]} as a
    sequence of fused GEMVs, every matrix distinct (3.17 GB of packed weight in total).

    After the timed passes of a schedule, what the buffers hold (the last layer's outputs) is
    compared with single-call GEMVs on the inputs the device had.  `oracle` (the tests pass the CPU
    oracle module; the benchmark itself never does) adds the same comparison against
    oracle.np_linear over the oracle-decompressed weights of the last layer."""
    import torch

    shapes = [(hidden, hidden)] * 4 + [(ffn, hidden), (hidden, ffn)]
    g = torch.Generator(device=device)
    g.manual_seed(9)
    xs = {k: torch.randn((m_rows, k), generator=g, device=device, dtype=torch.float32).to(torch.float16) for k in (hidden, ffn)}
    ys = [torch.empty((m_rows, n), dtype=torch.float16, device=device) for n, _ in shapes]  # one per role
    mats = []
    seed = 1000
    for layer in range(n_layers):
        for n_out, k_in in shapes:
            seed += 1
            mats.append((n_out, k_in) + tuple(pack_weight(make_weight(n_out, k_in, seed, False, device))))
        if layer % 7 == 6:
            log(f"  stack: packed {layer + 1}/{n_layers} layers")
    torch.cuda.synchronize()
    w_bytes = sum(n * k * (0.5 + 4.0 / GROUP) for n, k, *_ in mats)

    def one_pass(stream):
        for i, (n_out, k_in, p, s, b) in enumerate(mats):
            hip.call("gq_gemv_f16", xs[k_in].data_ptr(), m_rows, p.data_ptr(), s.data_ptr(), b.data_ptr(), 0,
                     ys[i % 6].data_ptr(), n_out, k_in, GROUP, stream)

    results = {"m": m_rows, "entries": len(mats), "weight_bytes": w_bytes}
    # (1) one launch per matrix, replayed from a HIP graph
    if modes is None or "per_launch_graph" in modes:
        one_pass(stream_handle())
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            one_pass(stream_handle())
        ms = time_launches(lambda _: graph.replay(), passes, warmup)
        results["per_launch_graph"] = {"us_per_pass": ms * 1e3, "weight_gbs": w_bytes / ms / 1e6,
                                       "hbm_frac": w_bytes / ms / 1e6 / HBM_PEAK_GBS,
                                       "roofline": hbm_roofline(one_shot_kernel_name(m_rows, ffn, hidden) + " (168 launches)", w_bytes, ms)}
    # (1b) the same stack with every weight in the default layout of LinearGQ (groups along the output
    # features), read from the derived copy a layer keeps after prepack_for_decode(): one launch of
    # gq_linear_knp_act_f16 per matrix replayed from a HIP graph, and the same entries as a sequence
    default_modes = ("default_layout_graph", "default_layout_sequence", "default_layout_two_entries_graph")
    if modes is None or any(mode in modes for mode in default_modes):
        # per layer: the six variables triples, packed [k_in, n_out / 64, 16]; roles q k v o up down
        kn_vars, seed = [], 5000
        for layer in range(n_layers):
            for n_out, k_in in shapes:
                seed += 1
                kn_vars.append(pack_weight(make_weight(k_in, n_out, seed, False, device)))
        torch.cuda.synchronize()

        def graph_of(one_pass):
            one_pass(stream_handle())
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                one_pass(stream_handle())
            return graph

        def knp(stream, x, w, y):
            hip.call("gq_linear_knp_act_f16", x.data_ptr(), m_rows, w.blob.data_ptr(), 0, y.data_ptr(), w.n_out, w.k_in, GROUP, 0, stream)

        if modes is None or "default_layout_graph" in modes or "default_layout_sequence" in modes:
            blobs = [hip.prepack_gemv_kn(*v) for v in kn_vars]
            if modes is None or "default_layout_graph" in modes:
                def one_pass_default(stream):
                    for i, w in enumerate(blobs):
                        knp(stream, xs[w.k_in], w, ys[i % 6])

                graph = graph_of(one_pass_default)
                ms = time_launches(lambda _: graph.replay(), passes, warmup)
                results["default_layout_graph"] = {"us_per_pass": ms * 1e3, "weight_gbs": w_bytes / ms / 1e6,
                                                   "hbm_frac": w_bytes / ms / 1e6 / HBM_PEAK_GBS,
                                                   "roofline": hbm_roofline("gemv_knp_kernel (168 launches)", w_bytes, ms)}
                del graph
            if modes is None or "default_layout_sequence" in modes:
                seq = hip.GemvSequence(device)
                for i, w in enumerate(blobs):
                    seq.add(xs[w.k_in], w, None, None, ys[i % 6], None, wait_previous=(i % 6) in (0, 3, 4, 5))
                ms = time_launches(lambda _: seq.run(), passes, warmup)
                torch.cuda.synchronize()
                results["default_layout_sequence"] = {"us_per_pass": ms * 1e3, "weight_gbs": w_bytes / ms / 1e6,
                                                      "hbm_frac": w_bytes / ms / 1e6 / HBM_PEAK_GBS, "status": int(seq.status.item()),
                                                      "roofline": hbm_roofline("gemv_knp_kernel (sequence of 168 entries)", w_bytes, ms)}
                del seq
            del blobs
            torch.cuda.empty_cache()
        if modes is None or "default_layout_two_entries_graph" in modes:
            # the decoder's data flow with two launches per layer: up | v | q | k stacked along the outputs
            # (LinearGQ.fuse: the variables side by side along the group axis) reads the layer input, and the
            # joint output product [down ; o] (LinearGQ.fuse_inputs: along the input features) reads
            # up's and v's results, which lie end to end, and writes the next layer's input
            first_w, out_w = [], []
            for layer in range(n_layers):
                q, k, v, o, up, down = (kn_vars[layer * 6 + role] for role in range(6))
                first_w.append(hip.prepack_gemv_kn(*(torch.cat([up[part], v[part], q[part], k[part]], dim=1).contiguous() for part in range(3))))
                # (scaled by 0.27 like the other layout's joint product: no normalisation layers here)
                both = [torch.cat([down[part], o[part]], dim=0).contiguous() for part in range(3)]
                out_w.append(hip.prepack_gemv_kn(both[0], (both[1].float() * 0.27).to(torch.float16), (both[2].float() * 0.27).to(torch.float16)))
            torch.cuda.synchronize()
            g.manual_seed(12)
            h_in = (torch.randn((m_rows, hidden), generator=g, device=device, dtype=torch.float32) * 0.1).to(torch.float16)
            wide = torch.empty((m_rows, ffn + 3 * hidden), dtype=torch.float16, device=device)
            h_out = [torch.empty((m_rows, hidden), dtype=torch.float16, device=device) for _ in range(2)]
            # (x of the joint product is the first ffn + hidden columns of the wide result, read where they lie: rows a
            # stride apart)

            def one_pass_two(stream):
                h = h_in
                for layer in range(n_layers):
                    knp(stream, h, first_w[layer], wide)
                    h = h_out[layer % 2]
                    hip.call("gq_linear_knp_strided_f16", wide.data_ptr(), wide.stride(0), m_rows, out_w[layer].blob.data_ptr(), 0,
                             h.data_ptr(), hidden, ffn + hidden, GROUP, 0, stream)

            graph = graph_of(one_pass_two)
            ms = time_launches(lambda _: graph.replay(), passes, warmup)
            torch.cuda.synchronize()
            finite = bool(torch.isfinite(h_out[(n_layers - 1) % 2].float()).all().item())
            results["default_layout_two_entries_graph"] = {
                "us_per_pass": ms * 1e3, "weight_gbs": w_bytes / ms / 1e6, "hbm_frac": w_bytes / ms / 1e6 / HBM_PEAK_GBS,
                "finite": finite, "roofline": hbm_roofline("gemv_knp_kernel (56 launches)", w_bytes, ms)}
            if not finite:
                raise SystemExit("bench.py: the default-layout stack produced values that are not finite")
            del graph, first_w, out_w
        del kn_vars
        torch.cuda.empty_cache()
    # (2) the whole stack as one gq_gemv_sequence_f16 call, with the dependencies of a decoder layer
    # declared per entry.  Roles per layer, in `mats` order: q k v o up down.
    #   sequential block   q waits for the previous layer, k and v share its input, then o, up and
    #                      down each wait for their predecessor (4 device-wide waits per layer)
    #   parallel block     attention and feed-forward read the same layer input (the 6B model of
    #                      these shapes is built that way): order q k v up o down; q waits for the
    #                      previous layer, o for v (up streams meanwhile), down for up
    #   ... fused qkv       the parallel block with q, k, v as one 12288 x 4096 entry: 112 entries per pass
    #   decoder data flow  the fused-qkv, ffn-first schedule with every entry reading what its predecessor
    #                      wrote (results travel through the kernel's tagged exchange: no reported completion)
    #   no waits           no dependencies: the streaming rate of the kernel alone, not a decoder
    def sequential(seq):
        for i, (n_out, k_in, p, s, b) in enumerate(mats):
            seq.add(xs[k_in], p, s, b, ys[i % 6], None, wait_previous=(i % 6) in (0, 3, 4, 5))

    def parallel(seq):
        last = None
        for layer in range(n_layers):
            idx = {}
            for role in (0, 1, 2, 4, 3, 5):
                n_out, k_in, p, s, b = mats[layer * 6 + role]
                wait_for = {0: last, 3: idx.get(2), 5: idx.get(4)}.get(role)
                idx[role] = seq.add(xs[k_in], p, s, b, ys[role], None, wait_for=wait_for)
            last = idx[5]

    def parallel_fused_qkv(seq):
        # the same, with q, k and v stacked into one [3 * hidden x hidden] entry (LinearGQ.fuse): 112 entries
        last = None
        for layer in range(n_layers):
            q, k, v, o, up, down = (mats[layer * 6 + role] for role in range(6))
            a = seq.add(xs[hidden], *fused_qkv[layer], y_qkv, None, wait_for=last)
            b_ = seq.add(xs[hidden], *up[2:], ys[4], None)
            seq.add(xs[hidden], *o[2:], ys[3], None, wait_for=a)
            last = seq.add(xs[ffn], *down[2:], ys[5], None, wait_for=b_)

    def parallel_fused_qkv_ffn_first(seq):
        # the same dependencies, entries ordered up, qkv, down, o: each wait names an entry that is
        # two entries back, so another matrix streams while its result settles; only the step to
        # the next layer (which needs o and down, both at the end) is exposed
        last = None
        for layer in range(n_layers):
            q, k, v, o, up, down = (mats[layer * 6 + role] for role in range(6))
            b_ = seq.add(xs[hidden], *up[2:], ys[4], None, wait_for=last)
            a = seq.add(xs[hidden], *fused_qkv[layer], y_qkv, None)
            seq.add(xs[ffn], *down[2:], ys[5], None, wait_for=b_)
            last = seq.add(xs[hidden], *o[2:], ys[3], None, wait_for=a)

    def parallel_fused_qkv_ffn_first_streaming(seq):
        # the same schedule with every weight in the streaming layout (gq_gemv_prepack_f16): the same
        # bytes, stored as the contiguous 4608-byte blocks the kernel fetches
        last = None
        for layer in range(n_layers):
            w_qkv, w_o, w_up, w_down = prepacked[layer]
            b_ = seq.add(xs[hidden], w_up, None, None, ys[4], None, wait_for=last)
            a = seq.add(xs[hidden], w_qkv, None, None, y_qkv, None)
            seq.add(xs[ffn], w_down, None, None, ys[5], None, wait_for=b_)
            last = seq.add(xs[hidden], w_o, None, None, ys[3], None, wait_for=a)

    def free(seq):
        for i, (n_out, k_in, p, s, b) in enumerate(mats):
            seq.add(xs[k_in], p, s, b, ys[i % 6], None)

    def free_streaming(seq):
        # no dependencies, weights in the streaming layout, q k v fused: the ceiling of the kernel
        for layer in range(n_layers):
            w_qkv, w_o, w_up, w_down = prepacked[layer]
            seq.add(xs[hidden], w_up, None, None, ys[4], None)
            seq.add(xs[hidden], w_qkv, None, None, y_qkv, None)
            seq.add(xs[ffn], w_down, None, None, ys[5], None)
            seq.add(xs[hidden], w_o, None, None, ys[3], None)

    fused_qkv = [tuple(torch.cat([mats[layer * 6 + role][2 + part] for role in range(3)], dim=0).contiguous()
                       for part in range(3)) for layer in range(n_layers)]
    y_qkv = torch.empty((m_rows, 3 * hidden), dtype=torch.float16, device=device)
    prepacked = [(hip.prepack_gemv(*fused_qkv[layer]),) + tuple(hip.prepack_gemv(*mats[layer * 6 + role][2:]) for role in (3, 4, 5))
                 for layer in range(n_layers)]
    # the decoder schedule with DATA flowing through every wait: up and qkv read the layer input h,
    # down reads up's output, o reads 4096-wide rows out of qkv's output, and o's output is the next
    # layer's h.  (h starts small: without normalisation layers every layer multiplies it by 1.6.)
    g.manual_seed(11)
    h0 = (torch.randn((m_rows, hidden), generator=g, device=device, dtype=torch.float32) * 1e-3).to(torch.float16)
    y_o2 = [torch.empty((m_rows, hidden), dtype=torch.float16, device=device) for _ in range(2)]

    def v_rows(t):
        return t.view(-1)[2 * hidden : 2 * hidden + m_rows * hidden].view(m_rows, hidden)

    def data_flow(seq, streaming=True):
        h, last = h0, None
        for layer in range(n_layers):
            if streaming:
                w_qkv, w_o, w_up, w_down = ((w, None, None) for w in prepacked[layer])
            else:
                w_qkv, w_o, w_up, w_down = fused_qkv[layer], mats[layer * 6 + 3][2:], mats[layer * 6 + 4][2:], mats[layer * 6 + 5][2:]
            b_ = seq.add(h, *w_up, ys[4], None, wait_for=last)
            a = seq.add(h, *w_qkv, y_qkv, None)
            seq.add(ys[4], *w_down, ys[5], None, wait_for=b_)
            last = seq.add(v_rows(y_qkv), *w_o, y_o2[layer % 2], None, wait_for=a)
            h = y_o2[layer % 2]

    # The parallel block as the model computes it: the next layer reads attention output PLUS
    # feed-forward output, h' = W_o v + W_down up, which is ONE product [W_down | W_o] [up ; v] with
    # the two weights side by side along their input features and x = the results of `up` and of the
    # first third of a v|q|k projection, end to end in memory (batch 1: rows of x must be
    # contiguous).  Three entries per layer, 84 per pass, the same weight bytes; every entry reads
    # what earlier entries wrote, and the step to the next layer waits for all of the layer.
    joint = None
    h0_joint = h0 * 100.0
    # ... and with up, v, q and k, which all read the layer input, stacked into one 28672-row entry
    # (LinearGQ.fuse) in front of it: two entries per layer, 56 per pass.
    joint_modes = ("sequence_decoder_data_flow_joint_output_streaming_layout", "sequence_decoder_data_flow_two_entries_streaming_layout")
    if m_rows == 1 and (modes is None or any(mode in modes for mode in joint_modes)):
        joint = {"w": [], "plain": None, "y": [torch.empty((1, hidden), dtype=torch.float16, device=device) for _ in range(2)],
                 "both": torch.empty((1, ffn + 3 * hidden), dtype=torch.float16, device=device)}
        for layer in range(n_layers):
            q, k, v, o, up, down = (mats[layer * 6 + role][2:] for role in range(6))
            vqk = tuple(torch.cat([v[part], q[part], k[part]], dim=0).contiguous() for part in range(3))
            out = [torch.cat([down[part], o[part]], dim=1).contiguous() for part in range(3)]
            # without normalisation layers the joint product would multiply the layer input by 3.7 per layer
            # (the four-entry schedule: by 1.6) and overflow fp16 after a dozen layers: scale the weight, i.e.
            # its scales and biases, by 0.27
            out = (out[0], (out[1].float() * 0.27).to(torch.float16), (out[2].float() * 0.27).to(torch.float16))
            first = tuple(torch.cat([up[part], vqk[part]], dim=0).contiguous() for part in range(3))
            joint["w"].append((prepacked[layer][2], hip.prepack_gemv(*vqk), hip.prepack_gemv(*out), hip.prepack_gemv(*first)))
            if layer == n_layers - 1:
                joint["plain"] = (up, vqk, out)

    def data_flow_joint_output(seq):
        h, last = h0_joint, None
        for layer in range(n_layers):
            w_up, w_vqk, w_out, _ = joint["w"][layer]
            seq.add(h, w_up, None, None, joint["both"][:, :ffn], None, wait_for=last)
            a = seq.add(h, w_vqk, None, None, joint["both"][:, ffn:], None, wait_for=last)
            h = joint["y"][layer % 2]
            last = seq.add(joint["both"][:, : ffn + hidden], w_out, None, None, h, None, wait_for=a)

    def data_flow_two_entries(seq):
        h, last = h0_joint, None
        for layer in range(n_layers):
            *_, w_out, w_first = joint["w"][layer]
            a = seq.add(h, w_first, None, None, joint["both"], None, wait_for=last)
            h = joint["y"][layer % 2]
            last = seq.add(joint["both"][:, : ffn + hidden], w_out, None, None, h, None, wait_for=a)

    for mode, fill in (("sequence_sequential_block", sequential), ("sequence_parallel_block", parallel),
                       ("sequence_parallel_block_fused_qkv", parallel_fused_qkv),
                       ("sequence_parallel_block_fused_qkv_ffn_first", parallel_fused_qkv_ffn_first),
                       ("sequence_parallel_block_fused_qkv_ffn_first_streaming_layout", parallel_fused_qkv_ffn_first_streaming),
                       ("sequence_decoder_data_flow", lambda seq: data_flow(seq, streaming=False)),
                       ("sequence_decoder_data_flow_streaming_layout", data_flow),
                       ("sequence_decoder_data_flow_joint_output_streaming_layout", data_flow_joint_output),
                       ("sequence_decoder_data_flow_two_entries_streaming_layout", data_flow_two_entries),
                       ("sequence_no_waits", free), ("sequence_no_waits_streaming_layout", free_streaming)):
        if (modes is not None and mode not in modes) or (mode in joint_modes and joint is None):
            continue
        seq = hip.GemvSequence(device)
        fill(seq)
        for y in ys + [y_qkv] + y_o2 + ([joint["both"]] + joint["y"] if joint else []):
            y.fill_(float("nan"))
        ms = time_launches(lambda _: seq.run(), passes, warmup)
        torch.cuda.synchronize()
        results[mode] = {"us_per_pass": ms * 1e3, "weight_gbs": w_bytes / ms / 1e6,
                         "hbm_frac": w_bytes / ms / 1e6 / HBM_PEAK_GBS, "status": int(seq.status.item()),
                         "waits_per_pass": sum(1 for e in seq.entries if e[10] > 0),
                         # batch 1, every weight in the streaming layout, every dependency carried by data: the
                         # data-flow kernel; anything else: the LDS-ring kernel
                         "roofline": hbm_roofline("gemv_mfma_kernel (one launch per entry)" if m_rows > 4 else
                                                  "gemv_flow_kernel" if m_rows == 1 and mode in FLOW_KERNEL_MODES else "gemv_stream_kernel",
                                                  w_bytes, ms)}
        # the timed passes computed something: what the buffers hold now (the last layer's outputs)
        # equals single-call GEMVs on the same weights and the inputs the device had
        worst = 0.0

        def worse(so_far, y, ref):
            # (a result that is not finite, or a reference that is all zero, makes the error NaN, and NaN stays)
            err = ((y.float() - ref.float()).abs().max() / ref.float().abs().max()).item()
            return err if not (err <= so_far) else so_far

        worst_oracle = 0.0

        def against_oracle(x_in, weight, y):
            import numpy as np

            w_dec = oracle.np_decompress(*(t.cpu().numpy() for t in weight))
            ref = oracle.np_linear(x_in.cpu().numpy(), w_dec)
            err = float(np.abs(y.cpu().numpy().astype(np.float64) - ref).max() / np.abs(ref).max())
            return err if not (err <= worst_oracle) else worst_oracle

        last = (n_layers - 1) * 6
        if mode in joint_modes:  # (the stacked first entry computes what up and v|q|k compute separately)
            both, h_last = joint["both"], joint["y"][(n_layers - 2) % 2]
            singles = ((h_last, joint["plain"][0], both[:, :ffn]), (h_last, joint["plain"][1], both[:, ffn:]),
                       (both[:, : ffn + hidden], joint["plain"][2], joint["y"][(n_layers - 1) % 2]))
            checks = ()
            for x_in, (p, s, b), y in singles:
                ref = torch.empty_like(y)
                hip.call("gq_gemv_f16", x_in.data_ptr(), 1, p.data_ptr(), s.data_ptr(), b.data_ptr(), 0, ref.data_ptr(),
                         y.shape[1], x_in.shape[1], GROUP, stream_handle())
                torch.cuda.synchronize()
                worst = worse(worst, y, ref)
                if oracle is not None:
                    worst_oracle = against_oracle(x_in, (p, s, b), y)
        elif "data_flow" in mode:
            h_last = y_o2[(n_layers - 2) % 2]
            checks = ((mats[last + 3][2:], v_rows(y_qkv), y_o2[(n_layers - 1) % 2]), (mats[last + 4][2:], h_last, ys[4]),
                      (mats[last + 5][2:], ys[4], ys[5]), (fused_qkv[n_layers - 1], h_last, y_qkv))
        else:
            checks = tuple((mats[last + role][2:], xs[mats[last + role][1]], ys[role]) for role in (3, 4, 5))
        for (p, s, b), x_in, y in checks:
            ref = torch.empty_like(y)
            hip.call("gq_gemv_f16", x_in.data_ptr(), m_rows, p.data_ptr(), s.data_ptr(), b.data_ptr(), 0, ref.data_ptr(),
                     y.shape[1], x_in.shape[1], GROUP, stream_handle())
            torch.cuda.synchronize()
            worst = worse(worst, y, ref)
            if oracle is not None:
                worst_oracle = against_oracle(x_in, (p, s, b), y)
        results[mode]["max_error_vs_single_call"] = worst
        if oracle is not None:
            results[mode]["max_error_vs_oracle"] = worst_oracle
        if not worst <= 2e-3 or results[mode]["status"] != 0 or not worst_oracle <= 1e-2:
            raise SystemExit(f"bench.py: stack mode {mode} (m={m_rows}) is wrong: error {worst} against single calls, "
                             f"{worst_oracle} against the oracle, status {results[mode]['status']}")
    # (3) the decoder's data flow with two launches per layer through the layer's entry point, gq_linear_p_act_f16 with the
    # weights' derived copies alone, replayed from a HIP graph: what serves batches of more than four rows, which the
    # persistent kernels do not take.  The weights of the two-entry schedule above: up | v | q | k stacked along the
    # outputs, then the joint output product [down | o] (scaled by 0.27: no normalisation layers here).
    mode = "streaming_layout_two_entries_graph"
    if modes is None or mode in modes:
        two = []
        for layer in range(n_layers):
            q, k, v, o, up, down = (mats[layer * 6 + role][2:] for role in range(6))
            first = tuple(torch.cat([up[part], v[part], q[part], k[part]], dim=0).contiguous() for part in range(3))
            out = [torch.cat([down[part], o[part]], dim=1).contiguous() for part in range(3)]
            out = (out[0], (out[1].float() * 0.27).to(torch.float16), (out[2].float() * 0.27).to(torch.float16))
            # (the calls hand over the copies alone; the variables of the last layer are kept for the check below)
            keep = layer == n_layers - 1
            two.append((first if keep else None, hip.prepack_gemv(*first), out if keep else None, hip.prepack_gemv(*out)))
        torch.cuda.synchronize()
        wide = torch.empty((m_rows, ffn + 3 * hidden), dtype=torch.float16, device=device)
        h_out = [torch.empty((m_rows, hidden), dtype=torch.float16, device=device) for _ in range(2)]
        # (x of the joint product is the first ffn + hidden columns of `wide`, read where they lie: rows a stride apart)
        joint_x = wide[:, : ffn + hidden]

        def layer_entry(stream, x, copy, y):
            hip.call("gq_linear_p_strided_f16", x.data_ptr(), x.stride(0), m_rows, 0, 0, 0, copy.blob.data_ptr(), 0, y.data_ptr(),
                     copy.n_out, copy.k_in, GROUP, 0, stream)

        def one_pass_two(stream):
            h = h0_joint
            for layer in range(n_layers):
                _, first_copy, _, out_copy = two[layer]
                layer_entry(stream, h, first_copy, wide)
                h = h_out[layer % 2]
                layer_entry(stream, joint_x, out_copy, h)

        one_pass_two(stream_handle())
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            one_pass_two(stream_handle())
        ms = time_launches(lambda _: graph.replay(), passes, warmup)
        torch.cuda.synchronize()
        names = [one_shot_kernel_name(m_rows, ffn + 3 * hidden, hidden), one_shot_kernel_name(m_rows, hidden, ffn + hidden)]
        kernel = " / ".join(dict.fromkeys(names)) + " (streaming layout; 56 launches)"
        results[mode] = {"us_per_pass": ms * 1e3, "weight_gbs": w_bytes / ms / 1e6, "hbm_frac": w_bytes / ms / 1e6 / HBM_PEAK_GBS,
                         "status": 0, "roofline": hbm_roofline(kernel, w_bytes, ms)}
        # the last layer's two results against single calls on the variables (and the oracle, when a test hands it over)
        worst, worst_oracle = 0.0, 0.0
        h_last = h_out[(n_layers - 2) % 2]
        first, _, out, _ = two[n_layers - 1]
        # (the single calls read a gathered copy of the joint product's x)
        for x_in, (p, s_, b), y in ((h_last, first, wide), (joint_x.contiguous(), out, h_out[(n_layers - 1) % 2])):
            assert x_in.is_contiguous() and x_in.shape[1] * 2 == p.shape[1] * p.shape[2] * 8 and y.shape[1] == p.shape[0]
            ref = torch.empty_like(y)
            hip.call("gq_gemv_f16", x_in.data_ptr(), m_rows, p.data_ptr(), s_.data_ptr(), b.data_ptr(), 0, ref.data_ptr(),
                     y.shape[1], x_in.shape[1], GROUP, stream_handle())
            torch.cuda.synchronize()
            err = ((y.float() - ref.float()).abs().max() / ref.float().abs().max()).item()
            worst = err if not (err <= worst) else worst
            if oracle is not None:
                import numpy as np

                ref64 = oracle.np_linear(x_in.cpu().numpy(), oracle.np_decompress(*(t.cpu().numpy() for t in (p, s_, b))))
                err = float(np.abs(y.cpu().numpy().astype(np.float64) - ref64).max() / np.abs(ref64).max())
                worst_oracle = err if not (err <= worst_oracle) else worst_oracle
        results[mode]["max_error_vs_single_call"] = worst
        if oracle is not None:
            results[mode]["max_error_vs_oracle"] = worst_oracle
        if not worst <= 2e-3 or not worst_oracle <= 1e-2:
            raise SystemExit(f"bench.py: stack mode {mode} (m={m_rows}) is wrong: error {worst} against single calls, "
                             f"{worst_oracle} against the oracle")
        del graph, two
        torch.cuda.empty_cache()
    return results


# ------------------------------------------------------------------------------------ output
HEADLINE_LIMIT = 4096  # bytes: the final stdout line must stay a line that a log capture keeps whole

# the decoder schedules of the stack, best first where several ran: what "decoder" means in the headline
DECODER_MODES = ("streaming_layout_two_entries_graph",
                 "sequence_decoder_data_flow_two_entries_streaming_layout", "sequence_decoder_data_flow_joint_output_streaming_layout",
                 "sequence_decoder_data_flow_streaming_layout", "sequence_decoder_data_flow",
                 "sequence_parallel_block_fused_qkv_ffn_first_streaming_layout", "sequence_parallel_block_fused_qkv_ffn_first")


def _row(r, frac_key):
    return {"m": r["m"], "n": r["n"], "k": r["k"], "us": round(r["us"], 1), "frac": round(r[frac_key], 3)}


def _stack_summary(r):
    """One record per batch of the 28-layer stack: the fastest decoder schedule that ran, the same
    kernel without dependencies, and one launch per matrix replayed from a graph."""
    out = {"m": r["m"]}
    ran = [(r[mode]["us_per_pass"], mode) for mode in DECODER_MODES if mode in r]
    if ran:
        us, mode = min(ran)
        out["decoder"] = {"us": round(us), "frac": round(r[mode]["hbm_frac"], 3), "kernel": r[mode]["roofline"]["kernel"],
                          "schedule": mode.replace("sequence_", "")}
    for key, mode in (("no_waits", "sequence_no_waits_streaming_layout"), ("per_launch_graph", "per_launch_graph"),
                      ("default_layout", "default_layout_graph"), ("default_layout_two_entries", "default_layout_two_entries_graph")):
        if mode in r:
            out[key] = {"us": round(r[mode]["us_per_pass"]), "frac": round(r[mode]["hbm_frac"], 3)}
    return out


def headline(result):
    """The line for stdout: the top-level keys as they are, `roofline`, `cpu_baseline` without its
    legs, and under `extra` one short record per benchmark shape (microseconds, fraction of the
    roofline that bounds it).  Everything else stays in the detail file."""
    extra = result.get("extra") or {}
    short = {k: extra[k] for k in ("detail_file", "gpu_equals_cpu_baseline_bits", "bench_wall_s") if k in extra}
    if any(k in extra for k in ("gemv", "linear_kn", "gemm")):
        short["weights"] = "every row rotates over > 600 MB of distinct packed weights"
    for key in ("decompress_transposed", "compress", "compress_f32"):
        if key in extra:
            short[key] = {"us": round(extra[key]["us"], 1), "frac": round(extra[key]["hbm_frac"], 3)}
    if "gemv" in extra:  # configuration 3 (+ the stack's third shape): fraction of HBM peak on the packed weight
        short["c3_gemv"] = [_row(r, "hbm_frac") for r in extra["gemv"]]
    if "linear_knp" in extra:  # the same shapes in the default layout of LinearGQ ([k_in, n_out]), from the derived copy
        short["c3_gemv_default_layout"] = [_row(r, "hbm_frac") for r in extra["linear_knp"] if r["m"] <= 16]
        short["c4_gemm_default_layout"] = [_row(r, "mfma_frac") for r in extra["linear_knp"] if r["m"] > 16]
    if "gemv_streaming_layout" in extra:  # configuration 3 with the weight's derived copy beside the variables
        short["c3_gemv_streaming_layout"] = [_row(r, "hbm_frac") for r in extra["gemv_streaming_layout"]]
    # (the default layout from the three variables as they are, `linear_kn`: in the detail file)
    if "gemm" in extra:  # configuration 4: fraction of the dense fp16 MFMA peak
        short["c4_gemm"] = [_row(r, "mfma_frac") for r in extra["gemm"]]
    if "gemm_streaming_layout" in extra:  # ... the same with the weight's derived copy beside the variables
        short["c4_gemm_streaming_layout"] = [_row(r, "mfma_frac") for r in extra["gemm_streaming_layout"]]
    if "stack" in extra:  # configuration 5: fraction of HBM peak on the packed weight
        short["c5_stack"] = [_stack_summary(r) for r in extra["stack"]]
    out = {k: v for k, v in result.items() if k not in ("extra", "cpu_baseline", "roofline")}
    roof = dict(result["roofline"])
    roof.pop("traffic_source", None)
    out["roofline"] = roof
    cpu = result.get("cpu_baseline")
    out["cpu_baseline"] = None if cpu is None else {k: v for k, v in cpu.items() if k != "legs"}
    out["extra"] = short
    return out


def emit(result, detail_path):
    """Detail to its file and to stderr, the headline as the last line of stdout."""
    if detail_path:
        try:
            os.makedirs(os.path.dirname(os.path.abspath(detail_path)), exist_ok=True)
            with open(detail_path, "w") as f:
                json.dump(result, f, indent=1)
            result["extra"]["detail_file"] = os.path.relpath(detail_path, ROOT) if os.path.abspath(detail_path).startswith(ROOT) else detail_path
        except OSError as e:  # (a read-only tree: the detail still goes to stderr)
            log(f"bench.py: could not write {detail_path}: {e}")
    log("detail: " + json.dumps(result))
    line = json.dumps(headline(result), separators=(",", ":"))
    if len(line) >= HEADLINE_LIMIT:  # never expected (a test holds the size on a full run's detail): drop the per-shape records
        slim = headline(result)
        slim["extra"] = {k: v for k, v in slim["extra"].items() if not isinstance(v, list)}
        line = json.dumps(slim, separators=(",", ":"))
    sys.stderr.flush()
    print(line, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--only", default="all", choices=["decompress", "compress", "gemv", "kn", "knp", "gemm", "stack", "all"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--stack-modes", default="",
                    help="comma-separated schedules of the 28-layer stack to run (default: all), e.g. for a profile of one kernel")
    ap.add_argument("--stack-batches", default="1,4,8", help="batch sizes of the stack runs")
    ap.add_argument("--gemv-shapes", default="", help="the single-launch rows after the benchmark's: these weights instead of the stack's two products (n_out x k_in, ...)")
    ap.add_argument("--gemv-batches", default="1,4,8", help="batches of those rows")
    ap.add_argument("--knp-shapes", default="", help="--only knp: decode rows on these weights instead (n_out x k_in, e.g. 4096x20480,28672x4096)")
    ap.add_argument("--knp-batches", default="1,8", help="decode batches of the knp rows")
    ap.add_argument("--detail", default=os.path.join(ROOT, "gpurun_out", "bench_detail.json"),
                    help="file for every figure of the run (the stdout line holds a summary); empty: no file")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 128 MiB device copy (known traffic) for scaling profiler byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU (no sharding, no collectives); use --gpus 1")

    import torch

    from popxl_addons import _gq_hip as hip

    hip.load()  # no CPU fallback: fails here if the HIP library is not built
    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP device visible")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    log(f"device: {torch.cuda.get_device_name(0)}")

    extra = {}
    t_begin = time.time()
    if args.calibrate_copy:
        n = 128 << 20
        srcs = [torch.zeros(n, dtype=torch.uint8, device=device) for _ in range(3)]
        dsts = [torch.empty(n, dtype=torch.uint8, device=device) for _ in range(3)]
        ms = time_launches(lambda i: dsts[i % 3].copy_(srcs[i % 3]), 30, 5)
        extra["calibrate_copy"] = {"bytes_read": n, "bytes_written": n, "us": ms * 1e3, "gbs": 2 * n / ms / 1e6}
        log(f"plain copy 128 MiB -> 128 MiB: {ms * 1e3:.1f} us, {2 * n / ms / 1e6:.0f} GB/s")
        del srcs, dsts
        torch.cuda.empty_cache()
    log("decompress 4096x16384 ...")
    dec = bench_decompress(hip, device, args.steps, args.warmup)
    log(f"  {dec['ms'] * 1e3:.1f} us/launch, {dec['gbs']:.0f} GB/s algorithmic ({dec['gbs'] / HBM_PEAK_GBS:.1%} of HBM peak)")

    cpu = None
    if not args.no_cpu_baseline:
        log("cpu baseline (numpy decompress) ...")
        cpu, cpu_out = cpu_baseline_decompress(dec["sets"])
        # the timed GPU path and the CPU baseline computed the same thing
        p, s, b, o = dec["sets"][0]
        hip.call("gq_decompress_f16", p.data_ptr(), s.data_ptr(), b.data_ptr(), o.data_ptr(), 4096, 256, 16, stream_handle())
        torch.cuda.synchronize()
        import numpy as np

        same = np.array_equal(o.cpu().numpy().view(np.uint16), cpu_out.view(np.uint16))
        extra["gpu_equals_cpu_baseline_bits"] = bool(same)
        log(f"  {cpu['value']:.3f} GB/s on 1 core; GPU output bit-identical: {same}")
        if args.only == "all":
            cpu["legs"] = cpu_baseline_legs()
            for leg in cpu["legs"]:
                log(f"  cpu: {leg['workload']}: {leg['seconds']:.3f} s, {leg['value']:.3f} {leg['unit']}")
    if args.only in ("all", "decompress"):
        # the same weight with the result transposed (dim=0 of the operator)
        outs_t = [torch.empty((16384, 4096), dtype=torch.float16, device=device) for _ in dec["sets"]]

        def step_t(i):
            p, s, b, _ = dec["sets"][i % len(outs_t)]
            hip.call("gq_decompress_f16_transposed", p.data_ptr(), s.data_ptr(), b.data_ptr(), outs_t[i % len(outs_t)].data_ptr(),
                     4096, 256, 16, stream_handle())

        run_until_steady(step_t)
        ms_t = time_launches(step_t, 100, 10)
        extra["decompress_transposed"] = {"rows": 4096, "cols": 16384, "us": ms_t * 1e3, "gbs": dec["bytes"] / ms_t / 1e6,
                                          "hbm_frac": dec["bytes"] / ms_t / 1e6 / HBM_PEAK_GBS,
                                          "roofline": hbm_roofline("decompress_transposed_tile_kernel", dec["bytes"], ms_t)}
        log(f"  transposed: {ms_t * 1e3:.1f} us, {dec['bytes'] / ms_t / 1e6:.0f} GB/s ({dec['bytes'] / ms_t / 1e6 / HBM_PEAK_GBS:.1%})")
        del outs_t
    del dec["sets"]
    torch.cuda.empty_cache()

    if args.only in ("compress", "all"):
        for key, f32 in (("compress", False), ("compress_f32", True)):
            r = bench_compress(hip, device, 100, 10, f32=f32)
            extra[key] = r
            log(f"  compress 4096x16384 from {r['input']}: {r['us']:.1f} us, {r['gbs']:.0f} GB/s algorithmic ({r['hbm_frac']:.1%} of HBM peak)")
            torch.cuda.empty_cache()
    if args.only in ("gemv", "all"):
        extra["gemv"] = []
        for n_out, k_in in ((4096, 4096), (16384, 4096), (4096, 16384)):
            for m in (1, 8):
                r = bench_linear(hip, device, "gq_gemv_f16", m, n_out, k_in, 200, 20,
                                 n_sets=sets_beyond_cache(n_out, k_in), kernel="gemv_sums_kernel" if m <= 2 else "gemv_mfma_kernel")
                extra["gemv"].append(r)
                log(f"  gemv m={m} [{n_out}x{k_in}]: {r['us']:.1f} us, {r['weight_gbs']:.0f} GB/s weights ({r['hbm_frac']:.1%})")
                torch.cuda.empty_cache()
    if args.only in ("gemv", "all"):
        # the same rows when the caller also holds the weight's derived copy in the streaming layout (what LinearGQ(dim=0)
        # does after prepack_for_decode()): the same kernel and the same bits, every load 1 KiB contiguous and read once
        extra["gemv_streaming_layout"] = []
        for n_out, k_in in ((4096, 4096), (16384, 4096), (4096, 16384)):
            for m in (1, 8):
                r = bench_linear(hip, device, "gq_linear_p_act_f16", m, n_out, k_in, 200, 20,
                                 n_sets=sets_beyond_cache(n_out, k_in),
                                 kernel=("gemv_sums_kernel" if m <= 2 else "gemv_mfma_kernel") + " (streaming layout)")
                extra["gemv_streaming_layout"].append(r)
                log(f"  gemv, streaming layout m={m} [{n_out}x{k_in}]: {r['us']:.1f} us, {r['weight_gbs']:.0f} GB/s weights ({r['hbm_frac']:.1%})")
                torch.cuda.empty_cache()
    if args.only in ("gemv", "all"):
        # the two products of a layer of the 56-entry stack schedule ([up | v | q | k] and [down | o]) as single launches, from
        # the copy; --gemv-shapes / --gemv-batches: other weights and batches
        shapes = [tuple(int(v) for v in s.split("x")) for s in args.gemv_shapes.split(",") if s] or [(28672, 4096), (4096, 20480)]
        extra["gemv_stack_products"] = []
        for n_out, k_in in shapes:
            for m in [int(v) for v in args.gemv_batches.split(",")]:
                r = bench_linear(hip, device, "gq_linear_p_act_f16", m, n_out, k_in, 200, 20, n_sets=sets_beyond_cache(n_out, k_in),
                                 kernel=one_shot_kernel_name(m, n_out, k_in) + " (streaming layout)")
                extra["gemv_stack_products"].append(r)
                log(f"  gemv, streaming layout m={m} [{n_out}x{k_in}]: {r['us']:.1f} us, {r['weight_gbs']:.0f} GB/s weights ({r['hbm_frac']:.1%}; {r['roofline']['kernel']})")
                torch.cuda.empty_cache()
    if args.only in ("kn", "all"):
        # the same shapes with the weight stored [k_in, n_out] and grouped along n_out: the default layout of LinearGQ
        extra["linear_kn"] = []
        for n_out, k_in in ((4096, 4096), (16384, 4096), (4096, 16384)):
            for m in (1, 8):
                r = bench_linear(hip, device, "gq_linear_kn_act_f16", m, n_out, k_in, 200, 20,
                                 n_sets=sets_beyond_cache(n_out, k_in), kernel="gemv_kn_kernel")
                extra["linear_kn"].append(r)
                log(f"  kn-layout gemv m={m} [{k_in}->{n_out}]: {r['us']:.1f} us, {r['weight_gbs']:.0f} GB/s weights ({r['hbm_frac']:.1%})")
                torch.cuda.empty_cache()
        r = bench_linear(hip, device, "gq_linear_kn_act_f16", 128, 16384, 4096, 60, 5, n_sets=sets_beyond_cache(16384, 4096), kernel="gemm_kn_tile_kernel")
        extra["linear_kn"].append(r)
        log(f"  kn-layout gemm m=128 [4096->16384]: {r['us']:.1f} us, {r['tflops']:.0f} TFLOP/s ({r['mfma_frac']:.1%} of fp16 dense peak)")
        torch.cuda.empty_cache()
    if args.only in ("kn", "knp", "all"):
        # ... and from the derived copy that a layer keeps after prepack_for_decode(): the kn streaming layout
        extra["linear_knp"] = []
        shapes = [tuple(int(v) for v in s.split("x")) for s in args.knp_shapes.split(",") if s] or [(4096, 4096), (16384, 4096), (4096, 16384)]
        for n_out, k_in in shapes:
            for m in [int(v) for v in args.knp_batches.split(",")]:
                r = bench_linear(hip, device, "gq_linear_knp_act_f16", m, n_out, k_in, 200, 20,
                                 n_sets=sets_beyond_cache(n_out, k_in), kernel="gemv_knp_kernel")
                extra["linear_knp"].append(r)
                log(f"  kn streaming layout gemv m={m} [{k_in}->{n_out}]: {r['us']:.1f} us, {r['weight_gbs']:.0f} GB/s weights ({r['hbm_frac']:.1%})")
                torch.cuda.empty_cache()
        # prefill batches from the same copy (configuration 4 in the default layout): the MFMA pipeline of the other layout
        for m in (() if args.knp_shapes else (128, 512, 2048)):
            r = bench_linear(hip, device, "gq_linear_knp_act_f16", m, 16384, 4096, 60, 5, n_sets=sets_beyond_cache(16384, 4096),
                             kernel="gemm_pipe2_kn_kernel")
            extra["linear_knp"].append(r)
            log(f"  kn streaming layout gemm m={m} [4096->16384]: {r['us']:.1f} us, {r['tflops']:.0f} TFLOP/s ({r['mfma_frac']:.1%} of fp16 dense peak)")
            torch.cuda.empty_cache()
    if args.only in ("gemm", "all"):
        extra["gemm"] = []
        for m in (128, 512, 2048):
            # (weights out of HBM at every batch: 17 distinct 16384 x 4096 weights, 641 MB of packed bytes)
            r = bench_linear(hip, device, "gq_gemm_f16", m, 16384, 4096, 60, 5, n_sets=sets_beyond_cache(16384, 4096), kernel="gemm_pipe2_kernel")
            extra["gemm"].append(r)
            log(f"  gemm m={m} [16384x4096]: {r['us']:.1f} us, {r['tflops']:.0f} TFLOP/s ({r['mfma_frac']:.1%} of fp16 dense peak)")
            torch.cuda.empty_cache()
        # the same three batches when the caller also holds the weight in the streaming layout (what LinearGQ(dim=0) does
        # after prepack_for_decode()): the same kernel and the same bits, the weight pieces 512 bytes contiguous
        extra["gemm_streaming_layout"] = []
        for m in (128, 512, 2048):
            r = bench_linear(hip, device, "gq_linear_p_act_f16", m, 16384, 4096, 60, 5, n_sets=sets_beyond_cache(16384, 4096),
                             kernel="gemm_pipe2_kernel (streaming layout)")
            extra["gemm_streaming_layout"].append(r)
            log(f"  gemm, streaming layout m={m} [16384x4096]: {r['us']:.1f} us, {r['tflops']:.0f} TFLOP/s ({r['mfma_frac']:.1%} of fp16 dense peak)")
            torch.cuda.empty_cache()
        # the stack's other layer shapes (4096 outputs: few tiles, where the choice of tile matters most) and the
        # batches between the GEMV's 16 rows and full GEMM tiles, through the entry that the layer calls
        extra["gemm_other_shapes"] = []
        for entry, m, n_out, k_in in (("gq_gemm_f16", 512, 4096, 4096), ("gq_gemm_f16", 512, 4096, 16384),
                                      ("gq_linear_act_ws_f16", 128, 4096, 4096), ("gq_linear_act_ws_f16", 128, 4096, 16384),
                                      ("gq_linear_act_ws_f16", 512, 4096, 16384),
                                      ("gq_linear_f16", 32, 4096, 4096), ("gq_linear_f16", 64, 16384, 4096)):
            r = bench_linear(hip, device, entry, m, n_out, k_in, 60, 5, n_sets=sets_beyond_cache(n_out, k_in),
                             kernel="gemm_pipe2_kernel" if entry != "gq_linear_f16" else "gemv_mfma_kernel passes / gemm_pipe2_kernel")
            r["entry"] = entry
            extra["gemm_other_shapes"].append(r)
            log(f"  {entry} m={m} [{n_out}x{k_in}]: {r['us']:.1f} us, {r['tflops']:.0f} TFLOP/s")
            torch.cuda.empty_cache()
    if args.only in ("stack", "all"):
        extra["stack"] = []
        modes = tuple(m for m in args.stack_modes.split(",") if m) or None
        for m in (int(v) for v in args.stack_batches.split(",")):
            # (a pass takes 0.5 to 1.6 ms; the first few dozen launches after a pause run up to 15 % slower
            # than the steady state, so they are warm-up)
            # (more than four batch rows: outside the persistent kernels, every entry is a launch of its own -- the
            # graph of single launches, one sequence, and the default layout's graphs say what there is to say)
            big = ("per_launch_graph", "sequence_parallel_block_fused_qkv_ffn_first", "default_layout_graph",
                   "default_layout_two_entries_graph", "streaming_layout_two_entries_graph")
            r = bench_stack(hip, device, m, passes=100, warmup=40, modes=modes if modes or m <= 4 else big)
            extra["stack"].append(r)
            for mode, v in r.items():
                if isinstance(v, dict) and "us_per_pass" in v:
                    log(f"  stack m={m} {mode}: {v['us_per_pass']:.0f} us/pass, {v['weight_gbs']:.0f} GB/s weights "
                        f"({v['hbm_frac']:.1%}) [{v['roofline']['kernel']}]")
            torch.cuda.empty_cache()
    extra["bench_wall_s"] = round(time.time() - t_begin, 1)

    traffic, traffic_commit = measured_traffic()
    result = {
        "metric": "decompress GB/s & %HBM peak; fused dequant-GEMV/GEMM GB/s, TFLOP/s, %roofline",
        "value": round(dec["gbs"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dec["ms"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "standalone int4->fp16 decompress, 4096x16384, group_size 64, N(0,0.02) + 0.1% outliers at 8 sigma, "
            "4 rotating buffer sets (688 MB > last-level cache)",
            "rows": 4096, "cols": 16384, "group_size": 64,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(dec["gbs"], 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(dec["gbs"] / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "traffic_source": None if traffic is None else f"profiles/decompress_kernel_4096x16384.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE at commit {traffic_commit})",
            "kernel": "decompress_kernel",
            "algorithmic_bytes_per_launch": dec["bytes"],
        },
        "cpu_baseline": cpu,
        "extra": extra,
    }
    emit(result, args.detail)


if __name__ == "__main__":
    main()
