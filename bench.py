"""Benchmark of the quantized Dense hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one forward pass of an int8-quantized Dense layer over one batch:
the fused abs-max activation quantizer followed by the int8 MFMA GEMM with the
de-scale epilogue, at the target shape M=4096, K=N=8192, bfloat16
activations (inputs and weights already resident in HBM).  `value` is
2*M*N*K / step time in TOP/s.  The int4 decode GEMV (K=N=8192, M in {1,4,16}),
the second half of the headline metric, is reported under `int4_gemv` with its own
HBM roofline (the layer's route: the strip-linear copy of the kernel, made once per layer).  `int8_gemm_sweep` holds the GEMM kernel's time over the
large-M sweep (M in {512, 2048, 4096, 8192} x K=N in {4096, 8192}, plus K=8192, N=28672),
`einsum_int8` the EinsumDense attention projections (batch 8, t in {1, 512});
`pack_unpack` the standalone pack_int4 / unpack_int4 kernels at 8192 x 8192 values on both axes,
`embedding_lookup` the quantized lookup of 32768 ids; `llama_decode_int4` is configuration 5 end to
end: a 32-layer Llama-style decoder with random float weights, `model.quantize("int4")` (seconds
reported), 128-token prompts and 128 greedy steps (tokens/s at batch 1 and 8, resident weight
bytes), `llama_decode_int8` the same with `model.quantize("int8")`.
The CPU oracle (a restatement of the reference's torch-CPU op sequence) is timed
on the host cores on a bounded sample as `cpu_baseline`.

Prints ONE JSON line.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

INT8_PEAK_TOPS = 5000.0  # MI355X dense int8, published (5.0 POP/s)
HBM_PEAK_GBS = 8000.0    # MI355X HBM3E, published (8 TB/s)

# Bytes crossing the L2 <-> memory boundary per launch: `rocprofv3 --pmc FETCH_SIZE` and
# `--pmc WRITE_SIZE` (KiB per dispatch) of this same command, each scaled by what the counter
# reads for a plain device copy of known size (FETCH_SIZE 0.50x, WRITE_SIZE 1.00x).  The
# figures are measured offline and kept in profiles/ with the command that produced them; this
# file reads them from there (kernel name -> bytes).  The file also records the SHA-256 of the
# kernel sources it was measured on (`_sources`); a figure whose kernel source has changed since
# is reported as null, with the file's name in `traffic_stale`, instead of being carried over.
# `python bench.py --sources-digest` prints the digests to record after a new profile.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_bytes.json")
CSRC = os.path.join(ROOT, "keras_amd", "csrc")
TRAFFIC_SOURCES = {  # key prefix -> the kernel's source files (all of them include k3q_common.h)
    "gemm_mfma": ["k3q_gemm_i8.hip"], "quantize_rows_vec": ["k3q_quantize.hip"], "gemv_w4s": ["k3q_gemv_w4s.hip"],
    "gemv_w8s": ["k3q_gemv_w8s.hip"], "pack_int4": ["k3q_pack.hip"], "unpack_int4": ["k3q_pack.hip"],
    "embedding_rows": ["k3q_embedding.hip"], "absmax_reduce": ["k3q_weight_quantize.hip"],
    "grouped_zp": ["k3q_weight_quantize.hip"],
}
TRAFFIC_STALE = set()


def sources_digest():
    import hashlib

    names = sorted({n for v in TRAFFIC_SOURCES.values() for n in v} | {"k3q_common.h"})
    out = {}
    for n in names:
        with open(os.path.join(CSRC, n), "rb") as f:
            out[n] = hashlib.sha256(f.read()).hexdigest()
    return out


def measured_traffic(key):
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    if key not in table:
        return None
    files = next((v for k, v in TRAFFIC_SOURCES.items() if key.startswith(k)), None)
    recorded = table.get("_sources", {})
    try:
        now = sources_digest()
    except OSError:
        return None
    for n in (files or []) + ["k3q_common.h"]:
        if files is None or recorded.get(n) != now.get(n):
            TRAFFIC_STALE.add(n if files is not None else key)
            return None
    return table[key]


def gemv_algorithmic_bytes(M, K, N, grouped, block=128):
    scales = 5 * (K // block) * N if grouped else 4 * N
    return K * (N // 2) + scales + 2 * M * K + 2 * M * N


# The GPU's clocks take tens of milliseconds of load to come up from idle (measured: the same
# GEMM runs 300 -> 240 us over its first 40 ms), and drop again while the host prepares the next
# section.  Every timed region below is therefore preceded by this much untimed work of the
# same kind, in addition to the --warmup steps.
CLOCK_SPIN_UP_S = 0.2


def spin_up(torch, fn, seconds=CLOCK_SPIN_UP_S):
    t_end = time.perf_counter() + seconds
    while time.perf_counter() < t_end:
        fn()
        torch.cuda.synchronize()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the host-side oracle timing")
    ap.add_argument("--no-decode", action="store_true", help="skip the end-to-end decoder measurement")
    ap.add_argument("--only", default="", help="comma list out of ceiling,sweep,einsum,gemv,gemv8,pack,wq,embed,decode,cpu: run the headline "
                    "step and only these further sections (for profiler runs); default: all")
    ap.add_argument("--sources-digest", action="store_true",
                    help="print the SHA-256 of the kernel sources (the `_sources` entry of profiles/hbm_traffic_bytes.json) and exit")
    args = ap.parse_args()
    if args.sources_digest:
        print(json.dumps(sources_digest(), indent=1))
        return
    only = set(filter(None, args.only.split(",")))
    unknown = only - {"none", "calib", "ceiling", "sweep", "einsum", "gemv", "gemv8", "pack", "wq", "embed", "decode", "cpu"}
    if unknown:
        sys.exit(f"bench.py: unknown section(s) {sorted(unknown)}")
    want = (lambda name: not only or name in only)
    if args.no_decode:
        want = (lambda name, w=want: name != "decode" and w(name))
    if args.no_cpu_baseline:
        want = (lambda name, w=want: name != "cpu" and w(name))
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the quantized Dense path has no multi-GPU leg "
                 f"(got --gpus {args.gpus}); its column-sharded form needs no exchange step")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device; none is visible")

    from keras_amd import _lib, ops as kops, quantizers as kq

    _lib.load()
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    g = torch.Generator().manual_seed(0)

    # ------------------------------------------------------------------ int8 Dense forward
    M, K, N = 4096, 8192, 8192
    limit = (6.0 / (K + N)) ** 0.5
    kernel_f = (torch.rand(K, N, generator=g) * 2 - 1) * limit  # glorot uniform
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
    wq, wscale = kq.abs_max_quantize(kernel_f, axis=0, to_numpy=True)  # one-time, host side
    wq = wq.to(dev)
    wscale_t = wscale.reshape(-1).to(torch.bfloat16).to(dev)
    # what an int8 layer keeps beside its stored kernel: the strip-linear copy, read by the decode
    # kernel and, as its B operand, by the tile GEMM (one-time, per layer)
    strip8 = kops.int8_strip_copy(wq)
    del kernel_f

    def step():
        q, s = kq.abs_max_quantize(x, axis=-1)
        return kops.int8_matmul(q, wq, a_scale=s, kernel_scale=wscale_t, out_dtype=torch.bfloat16,
                                strip=strip8, exact_epilogue=True)

    # W untimed warm-up steps, then exactly K timed steps.  The K steps are recorded once
    # into a HIP graph and replayed, so that the clock sees the kernels and not the Python
    # interpreter between them (the layer's forward is two launches).
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        step()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(args.steps):
                step()
    torch.cuda.synchronize()
    spin_up(torch, graph.replay)
    t0 = time.perf_counter()
    graph.replay()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    del graph
    ops_per_step = 2.0 * M * N * K
    value = ops_per_step / (ms_per_step * 1e-3) / 1e12

    # dominant kernel alone, HIP events on the stream it is launched on
    q, s = kq.abs_max_quantize(x, axis=-1)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2 * args.steps)]

    def gemm_burst():
        for _ in range(20):
            kops.int8_matmul(q, wq, a_scale=s, kernel_scale=wscale_t, out_dtype=torch.bfloat16,
                             strip=strip8, exact_epilogue=True)

    spin_up(torch, gemm_burst)
    for i in range(args.steps):
        ev[2 * i].record()
        kops.int8_matmul(q, wq, a_scale=s, kernel_scale=wscale_t, out_dtype=torch.bfloat16,
                         strip=strip8, exact_epilogue=True)
        ev[2 * i + 1].record()
    torch.cuda.synchronize()
    gemm_ms = sum(ev[2 * i].elapsed_time(ev[2 * i + 1]) for i in range(args.steps)) / args.steps
    gemm_tops = ops_per_step / (gemm_ms * 1e-3) / 1e12
    # the quantizer alone: a graph of K launches between two events (a launch of 20 us between events
    # of its own would be timed together with the host's pause before it)
    # The launches rotate over five copies of x (320 MiB, more than the 256 MiB memory-side cache holds).
    xs = [x] + [x.clone() for _ in range(4)]
    with torch.cuda.stream(side):
        kq.abs_max_quantize(x, axis=-1)
        qgraph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(qgraph, stream=side):
            for i in range(args.steps):
                kq.abs_max_quantize(xs[i % len(xs)], axis=-1)
    torch.cuda.synchronize()
    spin_up(torch, qgraph.replay, 0.05)
    ev[0].record()
    qgraph.replay()
    ev[1].record()
    torch.cuda.synchronize()
    quant_ms = ev[0].elapsed_time(ev[1]) / args.steps
    del qgraph, xs
    quant_bytes = M * K * 2 + M * K + M * 2

    # ------------------------------------------------------------------ counter calibration
    # only on request (--only ...,calib), for profiler runs: device copies of known size, so that
    # the same run that counts a kernel's FETCH_SIZE / WRITE_SIZE also counts these
    if "calib" in only:
        for mib in (64, 256):
            src_ = torch.randint(0, 255, (mib << 20,), dtype=torch.uint8, device=dev)
            for _ in range(5):
                dst_ = src_.clone()
            torch.cuda.synchronize()
            del src_, dst_

    # ------------------------------------------------------------------ matrix cores alone
    # What the int8 matrix cores sustain on this board with nothing else running: a loop of
    # v_mfma_i32_32x32x32_i8 on register-resident operands (bench_probes/libk3q_probe.so, a
    # measurement aid built beside this file, not part of the product library), about 50 ms per operand kind, clock read in-kernel.
    ceiling = None
    if want("ceiling"):
        import ctypes

        probe_path = os.path.join(ROOT, "bench_probes", "libk3q_probe.so")
        if os.path.exists(probe_path):
            probe = ctypes.CDLL(probe_path)
            probe.k3q_probe_mfma_i8_only.restype = ctypes.c_double
            probe.k3q_probe_mfma_i8_only.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
            pout = torch.zeros(4, dtype=torch.int64, device=dev)
            stream_h = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            ceiling = []
            for kind, label in ((0, "all-zero operands"), (1, "uniform random bytes"),
                                (2, "activation-like A (|a| < 32), uniform random B")):
                iters = 160000
                probe.k3q_probe_mfma_i8_only(kind, iters // 4, ctypes.c_void_p(pout.data_ptr()), stream_h)
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                n_ops = probe.k3q_probe_mfma_i8_only(kind, iters, ctypes.c_void_p(pout.data_ptr()), stream_h)
                e1.record()
                torch.cuda.synchronize()
                if n_ops <= 0:
                    sys.exit("bench.py: the MFMA-only probe did not launch")
                clk = pout.cpu().tolist()
                ceiling.append({"operands": label, "ms": round(e0.elapsed_time(e1), 2),
                                "tops": round(n_ops / (e0.elapsed_time(e1) * 1e-3) / 1e12, 1),
                                "clock_ghz": round(clk[0] / (clk[1] / 100e6) / 1e9, 3)})

    # ------------------------------------------------------------------ int8 GEMM sweep
    # the GEMM kernel alone (quantised activations given), bit-exact bfloat16 epilogue, HIP events
    # around bursts of launches on the stream they are issued on
    def kernel_us(fn, reps):
        spin_up(torch, lambda: [fn() for _ in range(10)], 0.05)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps * 1e3

    sweep = []
    for (Ks, Ns) in ((4096, 4096), (8192, 8192), (8192, 28672)) if want("sweep") else ():
        if (Ks, Ns) == (K, N):
            ws_, wp_, sc_ = wq, strip8, wscale_t
        else:
            ws_ = torch.randint(-127, 128, (Ks, Ns), device=dev, dtype=torch.int8)
            wp_ = kops.int8_strip_copy(ws_)
            sc_ = (torch.rand(Ns, device=dev) * 100 + 100).to(torch.bfloat16)
        for Ms in (512, 2048, 4096, 8192):
            xs = torch.randn(Ms, Ks, device=dev).to(torch.bfloat16)
            qs, ss = kq.abs_max_quantize(xs, axis=-1)
            us_ = kernel_us(lambda: kops.int8_matmul(qs, ws_, a_scale=ss, kernel_scale=sc_,
                                                     out_dtype=torch.bfloat16, strip=wp_,
                                                     exact_epilogue=True), 10 if Ms * Ns > 1 << 27 else 30)
            tops_ = 2.0 * Ms * Ns * Ks / us_ / 1e6
            sweep.append({"M": Ms, "K": Ks, "N": Ns, "us_per_launch": round(us_, 1),
                          "tops": round(tops_, 1), "frac": round(tops_ / INT8_PEAK_TOPS, 4)})
            del xs, qs, ss
        if (Ks, Ns) != (K, N):
            del ws_, wp_, sc_
            torch.cuda.empty_cache()

    # ------------------------------------------------------------------ EinsumDense int8
    # attention projections, d_model 4096, 32 heads x 128, batch 8, bfloat16; one layer call
    # (quantizer + matmul + de-scale) replayed from a HIP graph
    from keras_amd.layers import EinsumDense

    einsum = []
    for t_ in (1, 512) if want("einsum") else ():
        for eq, oshape, ishape in (("btd,dnh->btnh", (None, 32, 128), (8, t_, 4096)),
                                   ("btnh,nhd->btd", (None, 4096), (8, t_, 32, 128))):
            layer = EinsumDense(eq, oshape, dtype="bfloat16", device=dev)
            layer.build((None,) + ishape[1:])
            layer.quantize("int8")
            xe = torch.randn(*ishape, device=dev).to(torch.bfloat16)
            side = torch.cuda.Stream()
            with torch.cuda.stream(side):
                layer(xe)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    for _ in range(20):
                        layer(xe)
            torch.cuda.synchronize()
            us_ = kernel_us(graph.replay, 5) / 20
            Me = 8 * t_
            tops_ = 2.0 * Me * 4096 * 4096 / us_ / 1e6
            row = {"equation": eq, "batch": 8, "t": t_, "M": Me, "K": 4096, "N": 4096,
                   "us_per_call": round(us_, 2), "tops": round(tops_, 1)}
            if t_ == 1:  # decode-sized: bound by the int8 kernel's bytes
                row["roofline"] = {"bound": "hbm", "achieved": round(4096 * 4096 / us_ / 1e3, 1),
                                   "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                   "frac": round(4096 * 4096 / us_ / 1e3 / HBM_PEAK_GBS, 4)}
            else:
                row["roofline"] = {"bound": "mfma", "achieved": round(tops_, 1), "peak": INT8_PEAK_TOPS,
                                   "unit": "TOP/s", "frac": round(tops_ / INT8_PEAK_TOPS, 4)}
            einsum.append(row)
            del graph, layer, xe

    # ------------------------------------------------------------------ int4 decode GEMV
    Kg = Ng = 8192
    # 12 x 32 MiB packed kernels: more than the 256 MiB last-level cache
    n_rot = 12 if want("gemv") else 1
    packs = [torch.randint(-128, 128, (Kg, Ng // 2), generator=g, dtype=torch.int8).to(dev)
             for _ in range(n_rot)]
    # what a layer keeps per kernel for decode-sized calls, made once: the strip-linear copy
    strips = [kops.int4_strip_copy(pk, Ng) for pk in packs]
    pc_scale = (torch.rand(Ng, generator=g) + 0.5).to(torch.bfloat16).to(dev)
    gr_scale = (torch.rand(Kg // 128, Ng, generator=g) * 0.01 + 0.001).to(torch.bfloat16).to(dev)
    gr_zero = torch.randint(-8, 8, (Kg // 128, Ng), generator=g, dtype=torch.int8).to(dev)
    gr_params = kops.int4_strip_params(gr_scale, gr_zero, Kg, Ng, 128)
    gemv = []
    for Mg in (1, 4, 16) if want("gemv") else ():
        xg = torch.randn(Mg, Kg, generator=g).to(torch.bfloat16).to(dev)
        for grouped in (False, True):
            strip = kops.int4_strip_supported(Mg, Kg, Ng, 128 if grouped else None)

            def call(i):
                if strip:  # the route Dense._int4_call takes for these rows
                    return kops.int4_matmul_strip(xg, strips[i % n_rot], Ng,
                                                  kernel_scale=None if grouped else pc_scale,
                                                  gparams=gr_params if grouped else None,
                                                  block_size=128 if grouped else None)
                if grouped:
                    return kops.int4_matmul(xg, packs[i % n_rot], gr_scale, Ng, kernel_zero=gr_zero,
                                            block_size=128)
                return kops.int4_matmul(xg, packs[i % n_rot], pc_scale, Ng)

            # a HIP graph of back-to-back calls: decode loops are launch-bound from Python
            reps = 4 * n_rot
            side = torch.cuda.Stream()
            with torch.cuda.stream(side):
                for i in range(n_rot):
                    call(i)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    for i in range(reps):
                        call(i)
            torch.cuda.synchronize()
            spin_up(torch, graph.replay, 0.05)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(3):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / (3 * reps) * 1e3
            nbytes = gemv_algorithmic_bytes(Mg, Kg, Ng, grouped)
            gbs = nbytes / (us * 1e-6) / 1e9
            gemv.append({
                "M": Mg, "K": Kg, "N": Ng,
                "scheme": "grouped/128+zero" if grouped else "per-channel",
                "kernel": "gemv_w4s (strip-linear copy)" if strip else "gemv_w4_mfma (stored kernel)",
                "us_per_call": round(us, 2), "algorithmic_bytes": nbytes,
                "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                             "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                             "traffic": measured_traffic(
                                 ("gemv_w4s" if strip else "gemv_w4_mfma") + f"_M{Mg}_"
                                 + ("grouped" if grouped else "per_channel"))},
            })
            del graph
        del xg

    # ------------------------------------------------------------------ what reading costs
    # The same graph-node timing for a launch that only READS a kernel's bytes (libk3q_probe.so:
    # the decode kernels' access pattern without their arithmetic, best of a few grid sizes and
    # queue depths) and for a launch that does nothing: the decode kernels are compared with these.
    def graph_node_us(call, count, reps):
        side_ = torch.cuda.Stream()
        with torch.cuda.stream(side_):
            for i in range(count):
                call(i)
            graph_ = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph_, stream=side_):
                for i in range(reps):
                    call(i)
        torch.cuda.synchronize()
        spin_up(torch, graph_.replay, 0.05)
        e0_, e1_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0_.record()
        for _ in range(3):
            graph_.replay()
        e1_.record()
        torch.cuda.synchronize()
        return e0_.elapsed_time(e1_) / (3 * reps) * 1e3

    def load_stream_probe():
        import ctypes

        path = os.path.join(ROOT, "bench_probes", "libk3q_probe.so")
        if not os.path.exists(path):
            return None
        lib_ = ctypes.CDLL(path)
        lib_.k3q_probe_stream_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                               ctypes.c_void_p, ctypes.c_void_p]
        lib_.k3q_probe_empty.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        return lib_

    def read_reference(buffers, nbytes):
        """Best time per graph node of a pure read of `nbytes` from each of `buffers` in turn."""
        import ctypes

        lib_ = load_stream_probe()
        if lib_ is None:
            return None
        sink = torch.zeros(4096, dtype=torch.int32, device=dev)
        best = None
        for wgs, depth in ((256, 8), (256, 16), (512, 4), (512, 8), (1024, 4), (1024, 8)):
            if nbytes % (wgs * 8 * depth * 1024) or nbytes // (wgs * 8) < 2048 * depth:
                continue  # (the probe wants at least two rounds of whole KiB pieces per wave)
            def call(i):
                rc = lib_.k3q_probe_stream_read(ctypes.c_void_p(buffers[i % len(buffers)].data_ptr()), nbytes, wgs, depth,
                                                ctypes.c_void_p(sink.data_ptr()),
                                                ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
                if rc != 0:
                    sys.exit("bench.py: the read-only probe did not launch")
            us_ = graph_node_us(call, len(buffers), 4 * len(buffers))
            if best is None or us_ < best["us_per_launch"]:
                best = {"bytes": nbytes, "us_per_launch": round(us_, 2), "workgroups": wgs, "loads_in_flight_per_wave": depth,
                        "gbs": round(nbytes / us_ / 1e3, 1)}

        def nothing(i):
            lib_.k3q_probe_empty(ctypes.c_void_p(sink.data_ptr()),
                                 ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        best["empty_launch_us"] = round(graph_node_us(nothing, 4, 400), 2)
        return best

    read_ref4 = None
    if want("gemv"):
        read_ref4 = read_reference(strips, Kg * Ng // 2)
        if read_ref4:
            for row in gemv:
                row["frac_of_read_only_launch"] = round(read_ref4["us_per_launch"] / row["us_per_call"], 3)

    # ------------------------------------------------------------------ int8 decode forward
    # Dense int8 at decode sizes, K = N = 8192: quantizer + exact int8 matmul + bit-exact de-scale,
    # one launch from the strip-linear copy of the int8 kernel (x above 16 K values: a quantizer
    # launch first); 6 kernels of 64 MiB in rotation, each call a graph node
    gemv8 = []
    read_ref8 = None
    if want("gemv8"):
        n_rot8 = 6
        w8 = [torch.randint(-127, 128, (Kg, Ng), dtype=torch.int8, device=dev) for _ in range(n_rot8)]
        s8 = [kops.int8_strip_copy(w) for w in w8]
        del w8
        ks8 = (torch.rand(Ng, device=dev) * 50 + 50).to(torch.bfloat16)
        for M8 in (1, 8, 16):
            x8 = torch.randn(M8, Kg, device=dev).to(torch.bfloat16)
            reps = 4 * n_rot8
            side = torch.cuda.Stream()
            with torch.cuda.stream(side):
                for i in range(n_rot8):
                    kops.int8_dense_strip(x8, s8[i], Ng, ks8)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=side):
                    for i in range(reps):
                        kops.int8_dense_strip(x8, s8[i % n_rot8], Ng, ks8)
            torch.cuda.synchronize()
            spin_up(torch, graph.replay, 0.05)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(3):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / (3 * reps) * 1e3
            nbytes = Kg * Ng + 2 * M8 * Kg + 2 * M8 * Ng + 2 * Ng
            gbs = nbytes / (us * 1e-6) / 1e9
            gemv8.append({"M": M8, "K": Kg, "N": Ng, "kernel": "gemv_w8s (strip-linear copy)"
                          + ("" if kops.int8_strip_quantises_inside(M8, Kg, (-127, 127)) else " + quantize_rows_vec"),
                          "us_per_call": round(us, 2), "algorithmic_bytes": nbytes,
                          "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                                       "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                                       "traffic": measured_traffic(
                                           "gemv_w8s_M1" if kops.int8_strip_quantises_inside(M8, Kg, (-127, 127))
                                           else "gemv_w8s_prequantised")}})
            del graph, x8
        read_ref8 = read_reference(s8, Kg * Ng)
        if read_ref8:
            for row in gemv8:
                row["frac_of_read_only_launch"] = round(read_ref8["us_per_launch"] / row["us_per_call"], 3)
        del s8
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ pack / unpack int4
    # The standalone kernels at the config-2 kernel size (8192 x 8192 int4 values), along the last
    # axis (what Dense / EinsumDense store) and along axis 0; HBM-bound, 1.5 bytes per value (one
    # unpacked byte + half a packed one).  Cold: the calls rotate over five tensors of 64 MiB
    # (packing) or 32 MiB + 64 MiB of fresh output (unpacking), more than the 256 MiB memory-side
    # cache holds; each call is a graph node.
    pack_rows = []
    if want("pack"):
        n_val = Kg * Ng
        unpacked = [torch.randint(-8, 8, (Kg, Ng), dtype=torch.int8, device=dev) for _ in range(5)]
        for axis in (-1, 0):
            packed = [kq.pack_int4(u, axis=axis)[0] for u in unpacked]
            for name, call in (("pack_int4", lambda i: kq.pack_int4(unpacked[i % 5], axis=axis)),
                               ("unpack_int4", lambda i: kq.unpack_int4(packed[i % 5], Kg if axis == 0 else Ng, axis=axis))):
                us_ = graph_node_us(call, 5, 20)
                gbs_ = 1.5 * n_val / us_ / 1e3
                pack_rows.append({"op": name, "axis": axis, "values": n_val, "us_per_call": round(us_, 2),
                                  "algorithmic_bytes": int(1.5 * n_val),
                                  "roofline": {"bound": "hbm", "achieved": round(gbs_, 1), "peak": HBM_PEAK_GBS,
                                               "unit": "GB/s", "frac": round(gbs_ / HBM_PEAK_GBS, 4),
                                               "traffic": measured_traffic(
                                                   f"{name}_{'last_axis' if axis == -1 else 'axis0'}_64M")}})
            del packed
        del unpacked
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ weight quantizers on the device
    # What `quantize()` runs on a float32 kernel that lives on the device (the bits of the reference's
    # numpy path): per-column abs-max (int8 and per-channel int4) and the grouped min / max quantizer
    # (block 128), 8192 x 8192 float32; algorithmic bytes: 4 read + 1 written per weight.  The kernels
    # make two passes over x and memory sees both (`traffic`): a column's maximum needs the whole
    # column first, and the grouped kernel is bound by its arithmetic, not by the second read.
    # Rotating over two kernels of 256 MiB; eager calls, so host time per call counts as well.
    wq_rows = []
    if want("wq"):
        wf = [torch.randn(Kg, Ng, device=dev) * 0.02 for _ in range(2)]
        for name, key, call in (("abs_max_quantize axis=0 (int8)", "absmax_reduce_f32_8192x8192",
                                 lambda i: kq.abs_max_quantize(wf[i % 2], axis=0, to_numpy=True)),
                                ("abs_max_quantize_grouped_with_zero_point block 128 (int4)",
                                 "grouped_zp_f32_8192x8192_block128",
                                 lambda i: kq.abs_max_quantize_grouped_with_zero_point(wf[i % 2], 128, to_numpy=True))):
            call(0)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(20):
                call(i)
            e1.record()
            torch.cuda.synchronize()
            us_ = e0.elapsed_time(e1) / 20 * 1e3
            nb_ = 5 * Kg * Ng
            wq_rows.append({"op": name, "shape": [Kg, Ng], "us_per_call": round(us_, 1), "algorithmic_bytes": nb_,
                            "roofline": {"bound": "hbm", "achieved": round(nb_ / us_ / 1e3, 1), "peak": HBM_PEAK_GBS,
                                         "unit": "GB/s", "frac": round(nb_ / us_ / 1e3 / HBM_PEAK_GBS, 4),
                                         "traffic": measured_traffic(key)}})
        del wf
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ quantized embedding lookup
    # 32768 random ids into an int8 table of 32000 x 4096 with float32 per-row scales (what a
    # float32 or mixed_bfloat16 layer stores): 1 byte read and 4 written per element, plus the ids and
    # a scale per row; the output of a call (512 MiB) is more than the memory-side cache holds.
    embed_row = None
    if want("embed"):
        vocab_, dim_, count_ = 32000, 4096, 32768
        table_ = torch.randint(-127, 128, (vocab_, dim_), dtype=torch.int8, device=dev)
        tscale_ = (torch.rand(vocab_, device=dev) * 50 + 50)
        ids_ = torch.randint(0, vocab_, (count_,), device=dev)
        us_ = graph_node_us(lambda i: kops.embedding_lookup(ids_, table_, tscale_, dim_, check_ids=False), 2, 8)
        nbytes_ = count_ * dim_ * 5 + count_ * (8 + 4)
        embed_row = {"ids": count_, "vocab": vocab_, "dim": dim_, "table": "int8", "out": "float32",
                     "us_per_call": round(us_, 1), "algorithmic_bytes": nbytes_,
                     "roofline": {"bound": "hbm", "achieved": round(nbytes_ / us_ / 1e3, 1), "peak": HBM_PEAK_GBS,
                                  "unit": "GB/s", "frac": round(nbytes_ / us_ / 1e3 / HBM_PEAK_GBS, 4),
                                  "traffic": measured_traffic("embedding_rows_int8_32768x4096_f32")}}
        del table_, tscale_, ids_
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ end-to-end decode
    # Configuration 5 as written: a Llama-style 32-layer decoder (d_model 4096, 32 heads, SwiGLU
    # 14336, vocab 32000) built from the layer mirrors with random float weights (mixed_bfloat16:
    # float32 variables, bfloat16 compute; drawn on the device), converted with
    # `model.quantize("int4")` (grouped, block 128; the weight quantizers run on the device with the
    # bits of the reference's numpy path) or `model.quantize("int8")`, then 128 random prompt ids at
    # batch 1 and 8 and 128 greedy steps, prompt and decode steps replayed from HIP graphs.  Matmuls,
    # embedding lookup and LM head run the k3q kernels, and so do the harness's own normalisations,
    # RoPE + cache update + attention and the SwiGLU gate.
    decode = None
    decode_int8 = None
    if want("decode"):
        from keras_amd.decoder_harness import LlamaStyleDecoder

        w4_host = packs[0].cpu()
        del packs, strips
        torch.cuda.empty_cache()

        def decode_figures(mode):
            import warnings

            torch.cuda.synchronize()
            t0_ = time.perf_counter()
            model = LlamaStyleDecoder(max_len=256, dtype="mixed_bfloat16", device=dev, init_on_device=True)
            torch.cuda.synchronize()
            t1_ = time.perf_counter()
            with warnings.catch_warnings():
                warnings.simplefilter("ignore")  # (the norms have no quantized form: reported, not an error)
                report = model.quantize(mode)
            torch.cuda.synchronize()
            t2_ = time.perf_counter()
            torch.cuda.empty_cache()
            rows = []
            for batch in (1, 8):
                prompt = torch.randint(0, model.vocab, (batch, 128), generator=g)
                model.generate(prompt, 8)  # first-call set-up: the graphs of this shape are captured
                st = {}
                model.generate(prompt, 128, stats=st)
                rows.append({
                    "batch": batch, "prompt": 128, "steps": 128,
                    "prefill_ms": round(st["prefill_ms"], 2),
                    "decode_ms_per_step": round(st["decode_ms"] / st["decode_steps"], 3),
                    "tokens_per_s": round(batch * st["decode_steps"] / st["decode_ms"] * 1e3, 1),
                })
            resident = model.resident_bytes()
            out = {"policy": "mixed_bfloat16", "mode": mode, "init_float_weights_s": round(t1_ - t0_, 2),
                   "quantize_s": round(t2_ - t1_, 3), "layers_quantized": report.num_quantized,
                   # after a prompt and decode steps at both batch sizes: what the reference's layers
                   # store, and the copies this build keeps beside them for its kernels
                   "weights_resident_bytes": resident, "runs": rows}
            del model
            torch.cuda.empty_cache()
            return out

        decode = decode_figures("int4")
        # the same decoder with int8 layers (dynamic per-row activation quantisation)
        decode_int8 = decode_figures("int8")

    # ------------------------------------------------------------------ CPU baseline (oracle)
    cpu = None
    if want("cpu"):
        from oracle import keras_cpu_path as ref

        Mc = 2048  # bounded sample (about 10 s): 2048 rows of the same K = N = 8192 layer
        xc = x[:Mc].cpu()
        wq_c, ws_c = wq.cpu(), wscale.reshape(-1)
        ref.dense_int8_call(xc[:8], wq_c, ws_c, None, compute_dtype=torch.bfloat16)  # warm up
        t0 = time.perf_counter()
        ref.dense_int8_call(xc, wq_c, ws_c, None, compute_dtype=torch.bfloat16)
        cpu_s = time.perf_counter() - t0
        cpu = {
            "value": round(2.0 * Mc * N * K / cpu_s / 1e12, 5), "unit": "TOP/s",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle Dense int8 forward (torch-CPU op sequence of the reference), "
                      f"{Mc} of {M} rows, K=N={K}, one pass, {cpu_s:.1f} s; host has {os.cpu_count()} cpus",
        }
        # int4 decode GEMV on the host: unpack + float matmul per call, as the reference does
        w4 = w4_host if decode is not None else packs[0].cpu()
        x1 = torch.randn(1, Kg, generator=g).to(torch.bfloat16)
        ref.dense_int4_call(x1, w4, pc_scale.cpu().float(), Ng, compute_dtype=torch.bfloat16)
        t0 = time.perf_counter()
        for _ in range(3):
            ref.dense_int4_call(x1, w4, pc_scale.cpu().float(), Ng, compute_dtype=torch.bfloat16)
        g_s = (time.perf_counter() - t0) / 3
        cpu["int4_gemv"] = {"value": round(gemv_algorithmic_bytes(1, Kg, Ng, False) / g_s / 1e9, 3),
                            "unit": "GB/s", "sample": f"oracle Dense int4 per-channel, M=1, K=N={Kg}, 3 passes"}

    out = {
        "metric": "int8 GEMM TOPS (Dense int8 forward: quantize + GEMM + de-scale)",
        "value": round(value, 1),
        "unit": "TOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "clock_spin_up_s": CLOCK_SPIN_UP_S,  # untimed work before each timed region, besides warmup
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": f"Dense int8 forward M={M} K={K} N={N}, bf16 activations ~N(0,1), "
                               "glorot-uniform kernel quantized per channel, tile GEMM fed from the layer's strip-linear copy of the kernel"},
        "roofline": {"bound": "mfma", "achieved": round(gemm_tops, 1), "peak": INT8_PEAK_TOPS,
                     "unit": "TOP/s", "frac": round(gemm_tops / INT8_PEAK_TOPS, 4),
                     "traffic": measured_traffic("gemm_mfma_i8_M4096_K8192_N8192"), "kernel": "gemm_mfma<int8>",
                     "avg_launch_us": round(gemm_ms * 1e3, 1), "ops_per_launch": ops_per_step,
                     # share of what the matrix cores alone sustain on this board with random operands
                     "frac_of_mfma_only_random": (round(gemm_tops / ceiling[1]["tops"], 4) if ceiling else None),
                     "note": "int8 multiply-accumulate counted as 2 ops; peak is the published dense int8 figure"},
        "quantizer": {"kernel": "quantize_rows_vec", "avg_launch_us": round(quant_ms * 1e3, 1),
                      "roofline": {"bound": "hbm", "achieved": round(quant_bytes / (quant_ms * 1e-3) / 1e9, 1),
                                   "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                   "frac": round(quant_bytes / (quant_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                   "traffic": measured_traffic("quantize_rows_vec_bf16_4096x8192")}},
        "mfma_i8_only": ceiling,
        "int8_gemm_sweep": sweep,
        "einsum_int8": einsum,
        "int4_gemv": gemv,
        "read_only_launch_32MiB": read_ref4,
        "int8_decode_dense": gemv8,
        "read_only_launch_64MiB": read_ref8,
        "pack_unpack": pack_rows,
        "weight_quantizers": wq_rows,
        "embedding_lookup": embed_row,
        "llama_decode_int4": decode,
        "llama_decode_int8": decode_int8,
        "cpu_baseline": cpu,
    }
    if TRAFFIC_STALE:  # kernel sources that changed after their traffic figures were measured
        out["traffic_stale"] = sorted(TRAFFIC_STALE)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
