#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

Workload: the decode projections of one Llama-3-8B
layer at batch 1 -- Q8_0-quantize x[4096]; q_proj 4096x4096 Q8_0; ffn_gate and
ffn_up 14336x4096 Q4_K; Q8_0-quantize h[14336]; ffn_down 4096x14336 Q6_K -- with
synthetic N(0,0.02) weights and N(0,1) activations.  One step = one layer.  Steps
walk over `--layers` distinct weight sets (4.2 GB at 32) so that weights come from
HBM, not from the 256 MB Infinity Cache.  `value` = GGUF weight bytes streamed per
second over the timed steps (inputs resident in HBM, launches replayed from one
HIP graph so the host adds no per-kernel latency).

Prints ONE JSON line.  Extra objects:
  roofline     the dominant kernel of the timed step (Q4_K ffn_gate + ffn_up, 2 x 14336x4096, with SwiGLU and the
               quantizer of h in the same launch; --unfused-swiglu: the plain gate + up launch)
               timed alone with HIP events on the launch stream, algorithmic bytes / duration
               vs 8 TB/s
  kernels      the same figure for each GEMV shape, the lm_head and C1 shapes
  prefill      batch-512 Q4_K prefill matmul, int8 TOPS vs the 5.0 POPS peak
  moe          IQ4_XS grouped expert matmuls (8 experts, 64 tokens, top-2), weight GB/s
  moe_32_tokens  the same layer for a decode batch of 32 tokens (the few-token grouped kernel)
  moe_1_token    the same layer for one token (one GEMV launch per projection over the chosen experts);
                 the MoE legs call oxq_moe_forward_dev and are timed as replayed HIP graphs of six layers
  cpu_baseline the CPU restatement of the reference's fused rows on this host
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of `bench.py --traffic-probe`, each
# counter scaled by what it reads for a copy kernel of known size; the summary of those runs carries one
# `traffic-record:` line per kernel, keyed by the launch it was measured on (kernel instantiation, grid).  This
# run asks the library which launch it timed and reports the record only if the two agree.
TRAFFIC_SUMMARY = os.path.join("profiles", "hbm_traffic_gemv_gate_up_lm_head_prefill_pmc.txt")
INT8_PEAK_TOPS = 5000.0

Q4_0, Q8_0, Q4_K, Q6_K, IQ4_XS = 2, 8, 12, 14, 23


def row_bytes(t, n_cols):
    bs, bb = {2: (32, 18), 8: (32, 34), 12: (256, 144), 14: (256, 210), 23: (256, 136)}[t]
    return n_cols // bs * bb


def algorithmic_bytes(t, n_rows, n_cols):
    """Weight blocks + Q8_0 activation blocks + fp32 outputs of one GEMV launch."""
    return n_rows * row_bytes(t, n_cols) + n_cols // 32 * 34 + n_rows * 4


def last_launch():
    """What the library launched last on this thread: 'kernel<type,params> grid XxY block B'."""
    import ctypes as C
    from oxillama_amd import capi
    buf = C.create_string_buffer(256)
    capi.load().oxq_last_launch(buf, 256)
    return buf.value.decode()


def measured_traffic(launch):
    """HBM bytes per launch of `launch` from the tracked counter summary, or (None, reason)."""
    path = os.path.join(ROOT, TRAFFIC_SUMMARY)
    try:
        lines = [l for l in open(path) if l.startswith("traffic-record:")]
    except OSError:
        return None, f"{TRAFFIC_SUMMARY} is missing"
    for l in lines:
        fields = dict(kv.split("=", 1) for kv in l[len("traffic-record:"):].strip().split("; "))
        if fields.get("launch") == launch:
            return int(fields["hbm_bytes"]), f"{TRAFFIC_SUMMARY} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, copy-kernel scaled)"
    return None, f"no counter record for '{launch}' in {TRAFFIC_SUMMARY}: the launch changed since the counters were read"


def launch_phases(torch, dev, quant, linear, upload, synth):
    """Where the time of one decode GEMV launch goes: every wave of the kernel stamps the 100 MHz wall clock at
    kernel entry, after its first row batch is stored and after its last (the timestamping instantiation of the
    same kernels, oxq_set_gemv_phase_probe).  One launch at a time, a device synchronisation between launches,
    each launch on a weight set that no earlier launch touched (so HBM, not the Infinity Cache)."""
    import ctypes as C
    from oxillama_amd import capi
    lib = capi.load()
    H, F = 4096, 14336
    cap = 1 << 20
    buf = torch.zeros(cap // 8, dtype=torch.int64, device=dev)
    xq = torch.empty(H // 32 * 34, dtype=torch.uint8, device=dev)
    hq = torch.empty(F // 32 * 34, dtype=torch.uint8, device=dev)
    quant.quantize_q8_0_dev(torch.from_numpy(synth.normal_f32(1, H)).to(dev), xq)
    quant.quantize_q8_0_dev(torch.from_numpy(synth.normal_f32(2, F)).to(dev), hq)
    yH = torch.zeros(H, dtype=torch.float32, device=dev)
    yF, yF2 = torch.zeros(F, dtype=torch.float32, device=dev), torch.zeros(F, dtype=torch.float32, device=dev)
    hq_out = torch.empty(F // 32 * 34, dtype=torch.uint8, device=dev)
    k = {t: quant.HipKernel(t) for t in (Q4_0, Q8_0, Q4_K, Q6_K)}
    n_sets = 16
    gates = [upload(Q4_K, 2000 + i, F, H) for i in range(n_sets)]
    ups = [upload(Q4_K, 3000 + i, F, H) for i in range(n_sets)]
    downs = [upload(Q6_K, 4000 + i, H, F) for i in range(n_sets)]
    qs = [upload(Q8_0, 1000 + i, H, H) for i in range(n_sets)]
    c1 = [upload(Q4_0, 5000 + i, H, H) for i in range(n_sets)]
    cases = [
        ("gate + up + SwiGLU + quantize, one launch (2 x 14336x4096 Q4_K)", 2 * F * row_bytes(Q4_K, H),
         lambda i: linear.gate_up_swiglu_dev(Q4_K, gates[i], ups[i], xq, None, hq_out, F, H)),
        ("gate + up, one launch (2 x 14336x4096 Q4_K)", 2 * F * row_bytes(Q4_K, H),
         lambda i: k[Q4_K].matvec_q8_fused_multi_dev([gates[i], ups[i]], xq, [yF, yF2], F, H, accumulate=False)),
        ("gate alone (14336x4096 Q4_K)", F * row_bytes(Q4_K, H),
         lambda i: k[Q4_K].matvec_q8_fused_dev(gates[i], xq, yF, F, H, accumulate=False)),
        ("down (4096x14336 Q6_K)", H * row_bytes(Q6_K, F),
         lambda i: k[Q6_K].matvec_q8_fused_dev(downs[i], hq, yH, H, F, accumulate=False)),
        ("q_proj (4096x4096 Q8_0)", H * row_bytes(Q8_0, H),
         lambda i: k[Q8_0].matvec_q8_fused_dev(qs[i], xq, yH, H, H, accumulate=False)),
        ("C1 (4096x4096 Q4_0)", H * row_bytes(Q4_0, H),
         lambda i: k[Q4_0].matvec_q8_fused_dev(c1[i], xq, yH, H, H, accumulate=False)),
    ]
    kit = C.CDLL(os.path.join(ROOT, "oxillama_amd", "liboxq_benchkit.so"))
    kit.oxq_benchkit_read.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint, C.c_int, C.c_void_p]
    big = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
    sink = torch.zeros(1 << 16, dtype=torch.int32, device=dev)
    side = torch.cuda.Stream()

    def read_only(nbytes):
        """us per launch of the read-only kernel over nbytes, for three launch shapes (work groups x loads per lane and trip)."""
        nbytes = nbytes // 4096 * 4096
        nbuf, out = big.numel() // nbytes, []
        for blocks, unroll in ((512, 4), (2048, 2), (8192, 1)):
            def body():
                for i in range(32):
                    kit.oxq_benchkit_read(big.data_ptr() + (i % nbuf) * nbytes, sink.data_ptr(), nbytes, blocks, unroll,
                                          side.cuda_stream)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                body()
                side.synchronize()
                with torch.cuda.graph(g, stream=side):
                    body()
                best = 1e9
                for _ in range(3):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(side)
                    g.replay()
                    e1.record(side)
                    e1.synchronize()
                    best = min(best, e0.elapsed_time(e1))
            out.append((blocks, unroll, best * 1e3 / 32))
        return out

    def empty_launch_us():
        """us per launch of a kernel that does nothing (the read-only kernel over 0 bytes), 32 launches in a graph."""
        out = []
        for blocks in (512, 2048):
            def body():
                for _ in range(32):
                    kit.oxq_benchkit_read(big.data_ptr(), sink.data_ptr(), 0, blocks, 1, side.cuda_stream)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                body()
                side.synchronize()
                with torch.cuda.graph(g, stream=side):
                    body()
                best = 1e9
                for _ in range(3):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record(side)
                    g.replay()
                    e1.record(side)
                    e1.synchronize()
                    best = min(best, e0.elapsed_time(e1))
            out.append((blocks, best * 1e3 / 32))
        return out

    print("Launch phases of the decode GEMV kernels on MI355X: python bench.py --launch-phases")
    print("Every wave stamps the 100 MHz wall clock (10 ns steps) at kernel entry (t0), when its first row batch is stored (t1)")
    print("and when its last is (t2).  One launch at a time (device synchronised before each), %d launches per shape, each on" % n_sets)
    print("a weight set of its own (touched once before, %d sets = more than the 256 MB Infinity Cache for all but the two" % n_sets)
    print("4096x4096 shapes); times in us after the earliest t0 of the launch, median over the launches.")
    print("  entry: when waves enter the kernel (the dispatcher fills the chip);  first: first rows stored;  last: a wave's end.")
    print("  steady: sum over waves of (bytes the wave streams after its first batch) / (t2 - t1): the rate the waves sustain")
    print("  between ramp and tail;  span: last t2 - first t0;  whole: weight bytes / span.")
    print("  A launch that does nothing, back to back in a HIP graph (what every launch pays before its first wave runs and")
    print("  after its last has ended): " + ", ".join(f"{b_} work groups {us_:.2f} us" for b_, us_ in empty_launch_us()) + " per launch.")
    graph_us = {}
    for name, wbytes, fn in cases:
        rows, by_load = [], []
        for i in range(n_sets):  # first touch of a buffer pays for its page-table walks (66 MB: 17 us against 13)
            fn(i)
        torch.cuda.synchronize()
        for i in range(n_sets):
            buf.zero_()
            torch.cuda.synchronize()
            lib.oxq_set_gemv_phase_probe(buf.data_ptr(), cap)
            fn(i)
            lib.oxq_set_gemv_phase_probe(None, 0)
            torch.cuda.synchronize()
            launch = last_launch()
            raw = buf.cpu().numpy().reshape(-1, 4)
            raw = raw[raw[:, 0] != 0]
            t = raw[:, :3].astype(np.float64) / 100.0  # us
            # the compute unit a wave ran on: XCC_ID (bits 3:0 of the high word), shader engine / array / CU of HW_ID
            hw, xcc = raw[:, 3] & 0xFFFFFFFF, (raw[:, 3] >> 32) & 0xF
            cu_id = (xcc << 12) | (((hw >> 13) & 7) << 8) | (((hw >> 12) & 1) << 4) | ((hw >> 8) & 0xF)
            _, inv, cnt = np.unique(cu_id, return_inverse=True, return_counts=True)
            load = cnt[inv]  # waves of this launch on the wave's compute unit
            base = t[:, 0].min()
            t -= base
            dur = np.maximum(t[:, 2] - t[:, 1], 0.01)
            n_w = len(t)
            # a wave's bytes after its first batch: its share of the matrix minus one batch (shares are equal)
            share = wbytes / n_w
            first_share = share * (t[:, 1] - t[:, 0]).clip(0) / np.maximum(t[:, 2] - t[:, 0], 0.01)
            steady = float(((share - first_share) / dur).sum()) / 1e3  # GB/s
            rows.append([np.percentile(t[:, 0], 50), t[:, 0].max(), t[:, 1].min(), np.percentile(t[:, 1], 50),
                         np.percentile(t[:, 2], 10), np.percentile(t[:, 2], 50), t[:, 2].max(), steady, n_w])
            by_load.append({int(c): (int((load == c).sum()), float(np.median(t[load == c, 2])), float(t[load == c, 2].max()))
                            for c in np.unique(load)})
        r = np.median(np.array(rows), axis=0)
        span = r[6]
        print(f"\n{name}: {launch}, {int(r[8])} waves")
        print(f"  entry  median {r[0]:5.2f}  last {r[1]:5.2f}   first  earliest {r[2]:5.2f}  median {r[3]:5.2f}   "
              f"last  p10 {r[4]:5.2f}  median {r[5]:5.2f}  latest {r[6]:5.2f}")
        print(f"  steady {r[7]:7.0f} GB/s ({r[7] / 80:4.1f} % of 8 TB/s)   span {span:5.2f} us   whole {wbytes / span / 1e3:6.0f} GB/s "
              f"({wbytes / span / 1e3 / 80:4.1f} %)   ramp (median first) {r[3]:4.2f} us   tail (latest - median last) {r[6] - r[5]:4.2f} us")
        loads = sorted(set().union(*[d.keys() for d in by_load]))
        print("  by waves of the launch on the wave's compute unit: " + ";  ".join(
            "%d waves/CU: %d waves, last median %.2f latest %.2f" % (
                c, int(np.median([d[c][0] for d in by_load if c in d])), np.median([d[c][1] for d in by_load if c in d]),
                np.median([d[c][2] for d in by_load if c in d])) for c in loads))
        # the same launch timed the way the bench times it: 32 launches over the 16 sets in a HIP graph
        def body():
            for i in range(32):
                fn(i % n_sets)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            body()
            side.synchronize()
            with torch.cuda.graph(g, stream=side):
                body()
            best = 1e9
            for _ in range(3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(side)
                g.replay()
                e1.record(side)
                e1.synchronize()
                best = min(best, e0.elapsed_time(e1))
        print(f"  back to back in a HIP graph: {best * 1e3 / 32:.2f} us per launch, i.e. {best * 1e3 / 32 - span:.2f} us between one launch's "
              f"last store and the next one's first wave")
        print(f"  the same bytes with a kernel that only reads (16 bytes per lane, coalesced; graph of 32 launches over "
              f"distinct buffers): " + ", ".join(f"{b_}x{u_}: {us_:.2f} us" for b_, u_, us_ in read_only(wbytes)))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--layers", type=int, default=32, help="distinct weight sets the steps rotate over")
    ap.add_argument("--replays", type=int, default=7, help="times the K timed steps are replayed; the median is reported")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-extra-kernels", action="store_true")
    ap.add_argument("--no-moe", action="store_true")
    ap.add_argument("--f32-route", action="store_true",
                    help="also time the projections on the fp32-activation route (QuantKernel::gemv's own arithmetic); "
                         "the figures go to the --detail file, not to the result line")
    ap.add_argument("--detail", metavar="FILE", default=None,
                    help="write every leg's full record (launch names, sample descriptions, byte counts) as JSON to FILE; "
                         "the result line on stdout stays compact")
    ap.add_argument("--moe-tile-only", action="store_true",
                    help="run the 64-token MoE leg's grouped matmuls on the tile kernel alone (for profiles that set it "
                         "beside the few-token kernel)")
    ap.add_argument("--unfused-swiglu", action="store_true",
                    help="gate + up in one launch, SwiGLU + quantize in a second (default: all of it in one launch)")
    ap.add_argument("--fused-quantize", action="store_true",
                    help="decode step with the Q8_0 quantization done inside the GEMV kernels (3 launches per layer)")
    ap.add_argument("--launch-phases", action="store_true",
                    help="per-wave timestamps (kernel entry, first rows stored, last rows stored) of the decode GEMV "
                         "launches over distinct weight sets; prints the summary kept as profiles/gemv_launch_phases.txt")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="launch a 256 MiB copy kernel 3 times, then gate+up (one launch) over 8 distinct layers, "
                         "lm_head twice and the prefill matmul twice, and exit: the workload of the rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE runs (the copy kernel scales the counters)")
    ap.add_argument("--prefetch-probe", action="store_true",
                    help="the timed decode steps again with a small kernel on a second stream that, while a GEMV launch "
                         "runs, touches the first MB of the NEXT launch's weights (one dword per 128-byte line); prints "
                         "ms per step for several prefetch sizes and exits")
    ap.add_argument("--mfma-valu-probe", action="store_true",
                    help="time a kernel of f16 MFMAs and fp32 fmas on register operands in several proportions, one "
                         "work group of 8 waves per compute unit, and exit: how much vector work the matrix work hides")
    ap.add_argument("--token-sweep", action="store_true",
                    help="time oxq_gemm_q8_dev (the library's own choice of kernel) over 1..2048 token rows on the matrix "
                         "shapes of a 7-8 B model (Q4_K; Q6_K on the down shape), three rotating weight sets, replayed "
                         "graphs; prints one line per (format, shape, rows) with the launch the library took, and exits")
    ap.add_argument("--format-sweep", action="store_true",
                    help="time oxq_gemm_q8_dev on decode batches of 4 / 8 / 16 / 32 rows for all thirteen formats on the "
                         "gate and down shapes of a 7-8 B model: the library's choice and, beside it, the int8 tile "
                         "kernel forced (oxq_set_gemm_variant(99)); random valid blocks; prints one line per case, exits")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no collectives or sharding here)",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from oxillama_amd import linear, quant, synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    quant.init(0)
    info = quant.device_info()
    dev = torch.device("cuda:0")
    H, F = 4096, 14336
    L = max(1, args.layers)

    k_q8, k_q4k, k_q6k = quant.HipKernel(Q8_0), quant.HipKernel(Q4_K), quant.HipKernel(Q6_K)

    if args.token_sweep:
        sweep_stream = torch.cuda.Stream()
        for t, n, k in ((Q4_K, 4096, 4096), (Q4_K, 1024, 4096), (Q4_K, 14336, 4096), (Q4_K, 4096, 14336), (Q6_K, 4096, 14336)):
            kern = quant.HipKernel(t)
            sets = [torch.from_numpy(synth.weights(t, 100 + i, n, k)).to(dev) for i in range(3)]
            for m in (1, 2, 4, 5, 8, 16, 17, 32, 33, 64, 65, 128, 256, 384, 385, 512, 768, 1024, 2048):
                xq = torch.empty(m * (k // 32 * 34), dtype=torch.uint8, device=dev)
                quant.quantize_q8_0_dev(torch.from_numpy(synth.normal_f32(3, m * k)).to(dev), xq)
                y = torch.zeros(m * n, dtype=torch.float32, device=dev)
                wk = torch.empty(max(kern.gemm_workspace_bytes(m, n, k), 256), dtype=torch.uint8, device=dev)
                calls = [0]

                def call():
                    kern.gemm_q8_dev(sets[calls[0] % 3], xq, y, m, n, k, workspace=wk)
                    calls[0] += 1
                reps = 12
                g = torch.cuda.CUDAGraph()
                with torch.cuda.stream(sweep_stream):
                    call()
                    sweep_stream.synchronize()
                    with torch.cuda.graph(g, stream=sweep_stream):
                        for _ in range(reps):
                            call()
                    best = 1e9
                    for _ in range(3):
                        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        e0.record(sweep_stream)
                        g.replay()
                        e1.record(sweep_stream)
                        e1.synchronize()
                        best = min(best, e0.elapsed_time(e1) * 1e3 / reps)
                print(json.dumps({"format": {Q4_K: "Q4_K", Q6_K: "Q6_K"}[t], "n": n, "k": k, "rows": m, "us": round(best, 1),
                                  "us_per_row": round(best / m, 3), "launch": last_launch()}), flush=True)
            del sets
        return

    if args.format_sweep:
        from oxillama_amd import capi
        lib = capi.load()
        # (type id, name, weights per block, bytes per block, offsets of the block's f16 fields)
        formats = [(2, "Q4_0", 32, 18, (0,)), (3, "Q4_1", 32, 20, (0, 2)), (6, "Q5_0", 32, 22, (0,)), (7, "Q5_1", 32, 24, (0, 2)),
                   (8, "Q8_0", 32, 34, (0,)), (9, "Q8_1", 32, 36, (0, 2)), (10, "Q2_K", 256, 84, (80, 82)),
                   (11, "Q3_K", 256, 110, (108,)), (12, "Q4_K", 256, 144, (0, 2)), (13, "Q5_K", 256, 176, (0, 2)),
                   (14, "Q6_K", 256, 210, (208,)), (20, "IQ4_NL", 32, 18, (0,)), (23, "IQ4_XS", 256, 136, (0,))]
        sweep_stream = torch.cuda.Stream()
        rng = np.random.default_rng(5)
        for t, name, bs, bb, f16_at in formats:
            assert lib.oxq_block_size(t) == bs and lib.oxq_block_bytes(t) == bb, name
            kern = quant.HipKernel(t)
            for n, k in ((F, H), (H, F)):
                # every payload bit random, the f16 fields finite and small: any such bytes are a legal block
                blocks = rng.integers(0, 256, size=(256 * (k // bs), bb), dtype=np.uint8)
                for off in f16_at:
                    v = rng.uniform(0.005, 0.02, blocks.shape[0]).astype(np.float16)
                    blocks[:, off:off + 2] = v.view(np.uint8).reshape(-1, 2)
                one = torch.from_numpy(blocks.reshape(-1)).to(dev)
                sets = [one.repeat(n // 256) for _ in range(3)]
                for m in (4, 8, 16, 32):
                    xq = torch.empty(m * (k // 32 * 34), dtype=torch.uint8, device=dev)
                    quant.quantize_q8_0_dev(torch.from_numpy(synth.normal_f32(3, m * k)).to(dev), xq)
                    y = torch.zeros(m * n, dtype=torch.float32, device=dev)
                    wk = torch.empty(max(kern.gemm_workspace_bytes(m, n, k), 256), dtype=torch.uint8, device=dev)
                    row = {"format": name, "n": n, "k": k, "rows": m}
                    for variant, key in ((0, "us"), (99, "tile_kernel_us")):
                        lib.oxq_set_gemm_variant(variant)
                        calls = [0]

                        def call():
                            kern.gemm_q8_dev(sets[calls[0] % 3], xq, y, m, n, k, workspace=wk)
                            calls[0] += 1
                        g = torch.cuda.CUDAGraph()
                        with torch.cuda.stream(sweep_stream):
                            call()
                            sweep_stream.synchronize()
                            if variant == 0:
                                row["launch"] = last_launch()
                            with torch.cuda.graph(g, stream=sweep_stream):
                                for _ in range(12):
                                    call()
                            best = 1e9
                            for _ in range(3):
                                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                                e0.record(sweep_stream)
                                g.replay()
                                e1.record(sweep_stream)
                                e1.synchronize()
                                best = min(best, e0.elapsed_time(e1) * 1e3 / 12)
                        row[key] = round(best, 1)
                    lib.oxq_set_gemm_variant(0)
                    print(json.dumps(row), flush=True)
                del sets, one
        return

    if args.mfma_valu_probe:
        import ctypes as C
        kit = C.CDLL(os.path.join(ROOT, "oxillama_amd", "liboxq_benchkit.so"))
        kit.oxq_benchkit_mfma_valu.argtypes = [C.c_void_p, C.c_uint, C.c_int, C.c_int, C.c_int, C.c_void_p]
        iters = 4000
        rows = []
        for blocks in (info["compute_units"], 8):  # the whole chip busy, and 8 compute units of it
            buf = torch.zeros(max(blocks, 2) * 512, dtype=torch.float32, device=dev)
            for n_mfma, n_fma in ((0, 16), (0, 32), (2, 0), (2, 8), (2, 16), (2, 32)):
                best = 1e9
                for _ in range(3):
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    st = kit.oxq_benchkit_mfma_valu(buf.data_ptr(), blocks, iters, n_mfma, n_fma, None)
                    e1.record()
                    e1.synchronize()
                    assert st == 0, st
                    best = min(best, e0.elapsed_time(e1))
                # a SIMD runs two waves of the work group: 2 * iters trips
                rows.append({"work_groups": blocks, "mfma_32x32x16_f16_per_trip": n_mfma, "fma_f32_per_trip": n_fma,
                             "ns_per_trip_per_simd": round(best * 1e6 / (2 * iters), 1)})
        print(json.dumps({"probe": "mfma_valu", "waves_per_simd": 2, "trips": iters, "rows": rows}))
        return

    if args.traffic_probe:
        import ctypes as C
        kit = C.CDLL(os.path.join(ROOT, "oxillama_amd", "liboxq_benchkit.so"))
        kit.oxq_benchkit_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint, C.c_void_p]
        nbytes = 256 << 20
        src = torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(3):
            kit.oxq_benchkit_copy(src.data_ptr(), dst.data_ptr(), nbytes, 2048, None)
        torch.cuda.synchronize()
        del src, dst
        xq = torch.from_numpy(np.zeros(H // 32 * 34, dtype=np.uint8)).to(dev)
        quant.quantize_q8_0_dev(torch.from_numpy(synth.normal_f32(1, H)).to(dev), xq)
        yg = torch.zeros(F, dtype=torch.float32, device=dev)
        yu = torch.zeros(F, dtype=torch.float32, device=dev)
        hq_probe = torch.zeros(F // 32 * 34, dtype=torch.uint8, device=dev)
        for l in range(8):
            g, u = (torch.from_numpy(synth.weights(Q4_K, s0 + l, F, H)).to(dev) for s0 in (2000, 3000))
            torch.cuda.synchronize()
            k_q4k.matvec_q8_fused_multi_dev([g, u], xq, [yg, yu], F, H, accumulate=False)
            torch.cuda.synchronize()
            launches = {"gate_up": last_launch()}
            linear.gate_up_swiglu_dev(Q4_K, g, u, xq, None, hq_probe, F, H)
            torch.cuda.synchronize()
            launches["gate_up_swiglu"] = last_launch()
        V = 128256
        logits = torch.zeros(V, dtype=torch.float32, device=dev)
        for i in range(2):
            lm = torch.from_numpy(synth.weights(Q6_K, 6000 + i, V, H)).to(dev)
            torch.cuda.synchronize()
            k_q6k.matvec_q8_fused_dev(lm, xq, logits, V, H, accumulate=False)
            torch.cuda.synchronize()
            launches["lm_head"] = last_launch()
            del lm
        M = 512
        xsq = torch.empty(M * (H // 32 * 34), dtype=torch.uint8, device=dev)
        quant.quantize_q8_0_dev(torch.from_numpy(synth.normal_f32(3, M * H)).to(dev), xsq)
        ys = torch.zeros(M * F, dtype=torch.float32, device=dev)
        ws = torch.empty(k_q4k.gemm_workspace_bytes(M, F, H), dtype=torch.uint8, device=dev)
        for i in range(2):
            w = torch.from_numpy(synth.weights(Q4_K, 2100 + i, F, H)).to(dev)
            torch.cuda.synchronize()
            k_q4k.gemm_q8_dev(w, xsq, ys, M, F, H, workspace=ws)
            torch.cuda.synchronize()
            launches["prefill"] = last_launch()
        print(json.dumps({"traffic_probe": "done", "copy_bytes": nbytes, "launches": launches}), flush=True)
        return

    def upload(t, seed, n_rows, n_cols):
        return torch.from_numpy(synth.weights(t, seed, n_rows, n_cols)).to(dev)

    if args.launch_phases:
        launch_phases(torch, dev, quant, linear, upload, synth)
        return

    t0 = time.time()
    layers = []
    for l in range(L):
        layers.append({
            "q": upload(Q8_0, 1000 + l, H, H),
            "gate": upload(Q4_K, 2000 + l, F, H),
            "up": upload(Q4_K, 3000 + l, F, H),
            "down": upload(Q6_K, 4000 + l, H, F),
        })
    gen_s = time.time() - t0
    step_weight_bytes = H * row_bytes(Q8_0, H) + 2 * F * row_bytes(Q4_K, H) + H * row_bytes(Q6_K, F)

    x = torch.from_numpy(synth.normal_f32(1, H)).to(dev)
    h = torch.from_numpy(synth.normal_f32(2, F)).to(dev)
    xq = torch.empty(H // 32 * 34, dtype=torch.uint8, device=dev)
    hq = torch.empty(F // 32 * 34, dtype=torch.uint8, device=dev)
    yq = torch.zeros(H, dtype=torch.float32, device=dev)
    yg = torch.zeros(F, dtype=torch.float32, device=dev)
    yu = torch.zeros(F, dtype=torch.float32, device=dev)
    yd = torch.zeros(H, dtype=torch.float32, device=dev)

    stream = torch.cuda.Stream()

    def step(i):
        """One layer, four launches: quantize x; q_proj; ffn_gate + ffn_up + h = silu(gate) * up quantized
        to Q8_0 (one launch: a work group owns 32 rows of both matrices, one block of h); ffn_down on h.
        --unfused-swiglu: gate + up in one launch, SwiGLU + quantize in another (five launches).
        --fused-quantize lets the GEMV kernels quantize their fp32 input themselves (four
        launches, bit-identical results); measured slightly slower here: every work group then
        quantizes the whole vector into LDS before its first row, which costs more than the
        small launches it saves."""
        w = layers[i % L]
        if not args.fused_quantize:
            quant.quantize_q8_0_dev(x, xq)
            k_q8.matvec_q8_fused_dev(w["q"], xq, yq, H, H, accumulate=False)
            if args.unfused_swiglu:
                k_q4k.matvec_q8_fused_multi_dev([w["gate"], w["up"]], xq, [yg, yu], F, H, accumulate=False)
                linear.swiglu_quantize_dev(yg, yu, None, hq)
            else:
                linear.gate_up_swiglu_dev(Q4_K, w["gate"], w["up"], xq, None, hq, F, H)
            k_q6k.matvec_q8_fused_dev(w["down"], hq, yd, H, F, accumulate=False)
        else:
            k_q8.gemv_dev(w["q"], x, yq, H, H)
            k_q4k.gemv_multi_dev([w["gate"], w["up"]], x, [yg, yu], F, H)
            linear.swiglu_quantize_dev(yg, yu, h, None)
            k_q6k.gemv_dev(w["down"], h, yd, H, F)

    def capture(fn):
        """Record fn()'s launches on `stream` into a HIP graph."""
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            fn()  # eager once: first-use initialisation stays out of the capture
            stream.synchronize()
            with torch.cuda.graph(g, stream=stream):
                fn()
        return g

    def timed_replay(g):
        with torch.cuda.stream(stream):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            g.replay()
            e1.record(stream)
            e1.synchronize()
        return e0.elapsed_time(e1)  # ms

    if args.prefetch_probe:
        import ctypes as C
        kit = C.CDLL(os.path.join(ROOT, "oxillama_amd", "liboxq_benchkit.so"))
        kit.oxq_benchkit_touch.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_uint, C.c_void_p]
        side = torch.cuda.Stream()
        sink = torch.zeros(4096, dtype=torch.int32, device=dev)
        quant.quantize_q8_0_dev(x, xq)
        quant.quantize_q8_0_dev(h, hq)
        torch.cuda.synchronize()

        def launches_of(i):
            """The three weight-streaming launches of step i: (weights the launch reads, the call)."""
            w = layers[i % L]
            return [([w["q"]], lambda: k_q8.matvec_q8_fused_dev(w["q"], xq, yq, H, H, accumulate=False)),
                    ([w["gate"], w["up"]], lambda: linear.gate_up_swiglu_dev(Q4_K, w["gate"], w["up"], xq, None, hq, F, H)),
                    ([w["down"]], lambda: k_q6k.matvec_q8_fused_dev(w["down"], hq, yd, H, F, accumulate=False))]

        def steps_with_prefetch(n_steps, mb, blocks):
            seq = [l for i in range(n_steps) for l in launches_of(i)]
            for j, (_, call) in enumerate(seq):
                if mb and j + 1 < len(seq):
                    # while launch j runs: the head of launch j + 1's weights, on the second stream
                    side.wait_stream(stream)
                    nxt = seq[j + 1][0]
                    for t in nxt:
                        nb = min(t.numel(), (mb << 20) // len(nxt)) // 128 * 128
                        kit.oxq_benchkit_touch(t.data_ptr(), sink.data_ptr(), nb, blocks, side.cuda_stream)
                call()
            stream.wait_stream(side)

        rows = []
        for mb, blocks in ((0, 0), (2, 16), (4, 16), (8, 32), (16, 32), (16, 64), (32, 64)):
            g = capture(lambda: steps_with_prefetch(args.steps, mb, blocks))
            timed_replay(g)
            ms = sorted(timed_replay(g) for _ in range(5))[2] / args.steps
            rows.append({"prefetch_MB_per_launch": mb, "touch_work_groups": blocks, "ms_per_step": round(ms, 5)})
            print(json.dumps(rows[-1]), file=sys.stderr, flush=True)
        print(json.dumps({"probe": "prefetch", "steps": args.steps, "launches_per_step": 3,
                          "note": "activations pre-quantized (no quantize launch): compare the rows with each other, "
                                  "not with the default run", "rows": rows}))
        return

    # ---- the timed region: W warm-up steps, then exactly K steps ----------------------
    K, W = args.steps, args.warmup
    g_warm = capture(lambda: [step(i) for i in range(W)]) if W > 0 else None
    g_main = capture(lambda: [step(W + i) for i in range(K)])
    if g_warm is not None:
        with torch.cuda.stream(stream):
            g_warm.replay()
    torch.cuda.synchronize()
    # exactly K steps per replay, bracketed by synchronisation on both sides; the replay is repeated and the
    # MEDIAN is the reported figure (one replay of few steps is a sub-millisecond sample)
    R = max(1, args.replays)
    wall_ms, event_ms = [], []
    for _ in range(R):
        torch.cuda.synchronize()
        t_start = time.perf_counter()
        ev = timed_replay(g_main)  # HIP events on the launch stream, waits for the second one
        torch.cuda.synchronize()
        wall_ms.append((time.perf_counter() - t_start) * 1e3)
        event_ms.append(ev)
    ms_per_step = float(np.median(wall_ms)) / K
    value = step_weight_bytes / (ms_per_step * 1e-3) / 1e9
    timing = {"replays": R, "steps_per_replay": K, "reported": "median of the replays' host wall time / K",
              "ms_per_step_median": round(ms_per_step, 5), "ms_per_step_min": round(min(wall_ms) / K, 5),
              "ms_per_step_max": round(max(wall_ms) / K, 5),
              "ms_per_step_hip_events_median": round(float(np.median(event_ms)) / K, 5)}

    with torch.cuda.stream(stream):  # the per-kernel legs below read pre-quantized activations
        quant.quantize_q8_0_dev(x, xq)
        quant.quantize_q8_0_dev(h, hq)
        stream.synchronize()

    # ---- per-kernel figures: back-to-back launches of one shape over rotating weights ----
    def time_kernel(kern, t, mats, acts, out, n_rows, n_cols, launches=None):
        n = launches or max(len(mats), 64)
        n = -(-n // len(mats)) * len(mats)

        def body():
            for i in range(n):
                kern.matvec_q8_fused_dev(mats[i % len(mats)], acts, out, n_rows, n_cols, accumulate=False)
        g = capture(body)
        timed_replay(g)
        ms = min(timed_replay(g) for _ in range(3))
        us = ms * 1e3 / n
        ab = algorithmic_bytes(t, n_rows, n_cols)
        wb = n_rows * row_bytes(t, n_cols)
        return {"us_per_call": round(us, 3), "launches": n, "distinct_weight_sets": len(mats),
                "weight_GBps": round(wb / us / 1e3, 1), "algorithmic_GBps": round(ab / us / 1e3, 1),
                "frac_hbm_peak": round(ab / us / 1e3 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": ab}

    def time_pair():
        """ffn_gate + ffn_up of one layer in one launch, over all layers."""
        def body():
            for w in layers:
                k_q4k.matvec_q8_fused_multi_dev([w["gate"], w["up"]], xq, [yg, yu], F, H, accumulate=False)
        g = capture(body)
        timed_replay(g)
        us = min(timed_replay(g) for _ in range(3)) * 1e3 / L
        ab = 2 * F * row_bytes(Q4_K, H) + H // 32 * 34 + 2 * F * 4
        return {"us_per_call": round(us, 3), "launches": L, "distinct_weight_sets": L,
                "weight_GBps": round(2 * F * row_bytes(Q4_K, H) / us / 1e3, 1),
                "algorithmic_GBps": round(ab / us / 1e3, 1), "frac_hbm_peak": round(ab / us / 1e3 / HBM_PEAK_GBPS, 4),
                "algorithmic_bytes": ab}

    def time_pair_swiglu():
        """ffn_gate + ffn_up + SwiGLU + the Q8_0 quantizer of h in one launch, over all layers."""
        def body():
            for w in layers:
                linear.gate_up_swiglu_dev(Q4_K, w["gate"], w["up"], xq, None, hq, F, H)
        g = capture(body)
        timed_replay(g)
        us = min(timed_replay(g) for _ in range(3)) * 1e3 / L
        ab = 2 * F * row_bytes(Q4_K, H) + H // 32 * 34 + F // 32 * 34
        return {"us_per_call": round(us, 3), "launches": L, "distinct_weight_sets": L,
                "weight_GBps": round(2 * F * row_bytes(Q4_K, H) / us / 1e3, 1),
                "algorithmic_GBps": round(ab / us / 1e3, 1), "frac_hbm_peak": round(ab / us / 1e3 / HBM_PEAK_GBPS, 4),
                "algorithmic_bytes": ab}

    gate_up = [w["gate"] for w in layers] + [w["up"] for w in layers]
    pair = time_pair()
    pair_swiglu = time_pair_swiglu()
    with torch.cuda.stream(stream):  # the legs below read the quantized synthetic h again
        quant.quantize_q8_0_dev(h, hq)
        stream.synchronize()
    # the dominant kernel of the timed step, named by the launch the library actually makes for it
    with torch.cuda.stream(stream):
        if args.unfused_swiglu or args.fused_quantize:
            k_q4k.matvec_q8_fused_multi_dev([layers[0]["gate"], layers[0]["up"]], xq, [yg, yu], F, H, accumulate=False)
            dom, dom_name = pair, "ffn_gate + ffn_up (2 x 14336x4096 Q4_K) in one launch"
        else:
            linear.gate_up_swiglu_dev(Q4_K, layers[0]["gate"], layers[0]["up"], xq, None, hq, F, H)
            dom, dom_name = pair_swiglu, "ffn_gate + ffn_up (2 x 14336x4096 Q4_K) + SwiGLU + Q8_0 quantizer of h in one launch"
        dom_launch = last_launch()
        quant.quantize_q8_0_dev(h, hq)
        stream.synchronize()
    dom_traffic, traffic_source = measured_traffic(dom_launch)
    roofline = {"bound": "hbm", "kernel": dom_launch + ": " + dom_name,
                "achieved": dom["algorithmic_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": dom["frac_hbm_peak"],
                "traffic": dom_traffic, "traffic_source": traffic_source, "us_per_call": dom["us_per_call"],
                "algorithmic_bytes": dom["algorithmic_bytes"]}

    kernels = {"q4k_gate_plus_up_one_launch": pair, "q4k_gate_up_swiglu_one_launch": pair_swiglu,
               "q4k_gate_up_14336x4096": time_kernel(k_q4k, Q4_K, gate_up, xq, yg, F, H)}
    if not args.no_extra_kernels:
        kernels["q6k_down_4096x14336"] = time_kernel(k_q6k, Q6_K, [w["down"] for w in layers], hq, yd, H, F)
        kernels["q8_0_q_proj_4096x4096"] = time_kernel(k_q8, Q8_0, [w["q"] for w in layers], xq, yq, H, H)
        # same shape, one weight set only: resident in the Infinity Cache (not an HBM figure)
        kernels["q4k_gate_cache_resident"] = time_kernel(k_q4k, Q4_K, gate_up[:1], xq, yg, F, H, launches=64)
        k_q40 = quant.HipKernel(Q4_0)
        c1 = [upload(Q4_0, 5000 + i, H, H) for i in range(64)]
        kernels["c1_q4_0_4096x4096"] = time_kernel(k_q40, Q4_0, c1, xq, yq, H, H)
        # QuantKernel::gemv with the reference's own numerics (fp32 activations, oxq_gemv_f32_dev), same shapes
        def time_f32(kern, t, mats, xv, out, n_rows, n_cols):
            n = max(len(mats), 32)

            def body():
                for i in range(n):
                    kern.gemv_f32_dev(mats[i % len(mats)], xv, out, n_rows, n_cols)
            g = capture(body)
            timed_replay(g)
            us = min(timed_replay(g) for _ in range(3)) * 1e3 / n
            wb = n_rows * row_bytes(t, n_cols)
            return {"us_per_call": round(us, 3), "launches": n, "distinct_weight_sets": len(mats),
                    "weight_GBps": round(wb / us / 1e3, 1), "frac_hbm_peak": round((wb + 4 * n_cols + 4 * n_rows) / us / 1e3 / HBM_PEAK_GBPS, 4)}
        if args.f32_route:
            kernels["f32_route_q4k_gate_14336x4096"] = time_f32(k_q4k, Q4_K, [w["gate"] for w in layers], x, yg, F, H)
            kernels["f32_route_q6k_down_4096x14336"] = time_f32(k_q6k, Q6_K, [w["down"] for w in layers], h, yd, H, F)
            kernels["f32_route_q8_0_q_proj_4096x4096"] = time_f32(k_q8, Q8_0, [w["q"] for w in layers], x, yq, H, H)
            kernels["f32_route_c1_q4_0_4096x4096"] = time_f32(k_q40, Q4_0, c1, x, yq, H, H)
        del c1
        # a decode batch of 16 token rows on the Q4_K FFN shapes (oxq_gemm_q8_dev: the few-token kernel with k split
        # over work groups, then the reduction launch), over the layers' distinct weights
        def time_batch(kern, t, mats, m, n_rows, n_cols):
            xb = torch.from_numpy(synth.normal_f32(11, m * n_cols)).to(dev)
            xbq = torch.empty(m * (n_cols // 32 * 34), dtype=torch.uint8, device=dev)
            quant.quantize_q8_0_dev(xb, xbq)
            yb = torch.zeros(m * n_rows, dtype=torch.float32, device=dev)
            wsb = torch.empty(max(kern.gemm_workspace_bytes(m, n_rows, n_cols), 256), dtype=torch.uint8, device=dev)
            n = max(len(mats), 32)

            def body():
                for i in range(n):
                    kern.gemm_q8_dev(mats[i % len(mats)], xbq, yb, m, n_rows, n_cols, workspace=wsb)
            g = capture(body)
            timed_replay(g)
            us = min(timed_replay(g) for _ in range(3)) * 1e3 / n
            launch = last_launch()
            # the same calls on the int8-MFMA tile kernel (tuning knob 99: never the few-token kernel)
            from oxillama_amd import capi
            capi.load().oxq_set_gemm_variant(99)
            g2 = capture(body)
            timed_replay(g2)
            tile_us = min(timed_replay(g2) for _ in range(3)) * 1e3 / n
            capi.load().oxq_set_gemm_variant(0)
            wb = n_rows * row_bytes(t, n_cols)
            return {"us_per_call": round(us, 3), "token_rows": m, "launches": n, "distinct_weight_sets": len(mats),
                    "launch": launch, "weight_GBps": round(wb / us / 1e3, 1),
                    "frac_hbm_peak": round(wb / us / 1e3 / HBM_PEAK_GBPS, 4), "tile_kernel_us_per_call": round(tile_us, 3)}
        kernels["batch16_q4k_gate_14336x4096"] = time_batch(k_q4k, Q4_K, [w["gate"] for w in layers], 16, F, H)
        kernels["batch16_q4k_down_shape_4096x14336"] = time_batch(k_q4k, Q4_K, [w["gate"] for w in layers], 16, H, F)
        kernels["batch16_q6k_down_4096x14336"] = time_batch(k_q6k, Q6_K, [w["down"] for w in layers], 16, H, F)
        V = 128256
        lm = [upload(Q6_K, 6000 + i, V, H) for i in range(2)]
        logits = torch.zeros(V, dtype=torch.float32, device=dev)
        kernels["c3_lm_head_q6k_128256x4096"] = time_kernel(k_q6k, Q6_K, lm, xq, logits, V, H, launches=8)
        # ... followed by the sampler's candidate list: top_k = 40 (the GEMV launch and the two top-k launches), and the
        # argmax of greedy decoding as those launches and as the one launch in which the GEMV's waves select it
        def lm_then_list(top_k, one_launch):
            cand_v = torch.zeros(top_k, dtype=torch.float32, device=dev)
            cand_i = torch.zeros(top_k, dtype=torch.int32, device=dev)
            tws = torch.zeros(max(linear.topk_workspace_bytes(V, top_k), linear.lm_head_topk_workspace_bytes(Q6_K, V, H, top_k)) // 8 + 1,
                              dtype=torch.int64, device=dev)

            def body():
                for i in range(8):
                    if one_launch:
                        linear.lm_head_topk_dev(Q6_K, lm[i % 2], xq, logits, V, H, top_k, cand_v, cand_i, tws)
                    else:
                        k_q6k.matvec_q8_fused_dev(lm[i % 2], xq, logits, V, H, accumulate=False)
                        linear.topk_dev(logits, top_k, cand_v, cand_i, tws)
            g = capture(body)
            timed_replay(g)
            return round(min(timed_replay(g) for _ in range(3)) * 1e3 / 8, 2)
        kernels["c3_lm_head_then_candidates"] = {"top40_three_launches_us": lm_then_list(40, False),
                                                 "argmax_one_launch_us": lm_then_list(1, True),
                                                 "argmax_three_launches_us": lm_then_list(1, False)}
        del lm, logits

    # ---- prefill: 512 x 4096 activations times Q4_K 14336 x 4096 ---------------------------
    prefill = None
    if not args.no_prefill:
        M = 512
        xs = torch.from_numpy(synth.normal_f32(3, M * H)).to(dev)
        xsq = torch.empty(M * (H // 32 * 34), dtype=torch.uint8, device=dev)
        ys = torch.zeros(M * F, dtype=torch.float32, device=dev)
        wp = [layers[i % L]["gate"] for i in range(min(L, 8))]
        ws = torch.empty(max(k_q4k.gemm_workspace_bytes(M, F, H), 256), dtype=torch.uint8, device=dev)
        with torch.cuda.stream(stream):
            quant.quantize_q8_0_dev(xs, xsq)
            k_q4k.gemm_q8_dev(wp[0], xsq, ys, M, F, H, workspace=ws)
            stream.synchronize()
            prefill_launch = last_launch()
            reps = 8
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for i in range(reps):
                k_q4k.gemm_q8_dev(wp[i % len(wp)], xsq, ys, M, F, H, workspace=ws)
            e1.record(stream)
            e1.synchronize()
            gemm_us = e0.elapsed_time(e1) * 1e3 / reps
            e0.record(stream)
            for i in range(reps):
                quant.quantize_q8_0_dev(xs, xsq)
            e1.record(stream)
            e1.synchronize()
            quant_us = e0.elapsed_time(e1) * 1e3 / reps
        ops = 2 * M * F * H
        # the same shape in the other four formats (tile kernel, same workspace)
        others = {}
        for name, t in (("Q6_K", Q6_K), ("Q8_0", Q8_0), ("Q4_0", Q4_0), ("IQ4_XS", IQ4_XS)):
            kt = quant.HipKernel(t)
            wt = [upload(t, 8000 + i, F, H) for i in range(4)]
            wst = torch.empty(max(kt.gemm_workspace_bytes(M, F, H), 256), dtype=torch.uint8, device=dev)
            with torch.cuda.stream(stream):
                kt.gemm_q8_dev(wt[0], xsq, ys, M, F, H, workspace=wst)
                stream.synchronize()
                e0.record(stream)
                for i in range(4):
                    kt.gemm_q8_dev(wt[i], xsq, ys, M, F, H, workspace=wst)
                e1.record(stream)
                e1.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / 4
            others[name] = {"gemm_us": round(us, 2), "TOPS": round(ops / us / 1e6, 1)}
            del wt, wst
        # what the matrix cores deliver on a kernel of nothing but int8 MFMAs (register operands)
        import ctypes as C
        kit = C.CDLL(os.path.join(ROOT, "oxillama_amd", "liboxq_benchkit.so"))
        kit.oxq_benchkit_mfma_i8.argtypes = [C.c_void_p, C.c_uint, C.c_int, C.c_void_p]
        mf_blocks, mf_iters = 4096, 1024
        mf_out = torch.empty(mf_blocks * 256, dtype=torch.int32, device=dev)
        with torch.cuda.stream(stream):
            kit.oxq_benchkit_mfma_i8(mf_out.data_ptr(), mf_blocks, mf_iters, quant.HipKernel._stream())
            stream.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            kit.oxq_benchkit_mfma_i8(mf_out.data_ptr(), mf_blocks, mf_iters, quant.HipKernel._stream())
            e1.record(stream)
            e1.synchronize()
        mfma_only_tops = mf_blocks * 4 * mf_iters * 4 * 2 * 32 ** 3 / (e0.elapsed_time(e1) * 1e3) / 1e6
        # the int8 tile kernel on the same calls (tuning knob 99), beside the kernel the library chooses
        from oxillama_amd import capi as _capi
        _capi.load().oxq_set_gemm_variant(99)
        with torch.cuda.stream(stream):
            k_q4k.gemm_q8_dev(wp[0], xsq, ys, M, F, H, workspace=ws)
            stream.synchronize()
            e0.record(stream)
            for i in range(reps):
                k_q4k.gemm_q8_dev(wp[i % len(wp)], xsq, ys, M, F, H, workspace=ws)
            e1.record(stream)
            e1.synchronize()
        _capi.load().oxq_set_gemm_variant(0)
        tile_gemm_us = e0.elapsed_time(e1) * 1e3 / reps
        prefill = {"workload": "Q4_K 14336x4096 x Q8_0 acts 512x4096", "int8_ops": ops, "launch": prefill_launch,
                   "int8_tile_kernel_gemm_us": round(tile_gemm_us, 2),
                   "gemm_us": round(gemm_us, 2), "quantize_us": round(quant_us, 2),
                   "TOPS": round(ops / gemm_us / 1e6, 2), "peak_TOPS": INT8_PEAK_TOPS,
                   "frac_int8_peak": round(ops / gemm_us / 1e6 / INT8_PEAK_TOPS, 4),
                   "mfma_only_TOPS": round(mfma_only_tops, 1),
                   "frac_of_mfma_only": round(ops / gemm_us / 1e6 / mfma_only_tops, 4),
                   "same_shape_other_formats": others}

    # ---- C5: Mixtral-shaped IQ4_XS expert matmuls, 64 tokens, top-2 of 8 experts ------------
    moe_out = None
    moe_small = None
    moe_one = None
    if not args.no_moe:
        from oxillama_amd import moe
        E, TOPK = 8, 2

        def expert_set(seed, n_rows, n_cols):
            return torch.from_numpy(np.stack([synth.weights(IQ4_XS, seed + e, n_rows, n_cols) for e in range(E)])).to(dev)
        wg, wu, wd = expert_set(7000, F, H), expert_set(7100, F, H), expert_set(7200, H, F)
        stride = wg[0].numel()
        router = torch.from_numpy(synth.normal_f32(9, E * H, 0.05)).to(dev)
        types3 = (IQ4_XS, IQ4_XS, IQ4_XS)

        def moe_leg(NTOK, tile_only=False):
            from oxillama_amd import capi
            capi.load().oxq_set_gemm_variant(99 if tile_only else 0)  # 99: the tile kernel's own choice of shape
            try:
                return moe_leg_timed(NTOK)
            finally:
                capi.load().oxq_set_gemm_variant(0)

        def moe_leg_timed(NTOK):
            xt = torch.from_numpy(synth.normal_f32(7, NTOK * H)).to(dev)
            rows = NTOK * TOPK
            d_y = torch.empty(NTOK * H, dtype=torch.float32, device=dev)
            wsm = torch.empty(moe.moe_forward_workspace_bytes(types3, NTOK, TOPK, E, H, F), dtype=torch.uint8, device=dev)
            off_at = 2 * ((4 * rows + 255) & ~255)  # the workspace starts with experts | weights | offsets | ...

            def moe_step():
                moe.moe_forward_dev((IQ4_XS, wg, stride), (IQ4_XS, wu, stride), (IQ4_XS, wd, stride), E, router, xt, NTOK,
                                    TOPK, d_y, H, F, wsm)

            reps = 6
            with torch.cuda.stream(stream):
                moe_step()
                stream.synchronize()
                offsets = wsm[off_at:off_at + 4 * (E + 1)].cpu().numpy().view(np.int32)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(reps):
                    moe_step()
                e1.record(stream)
                e1.synchronize()
            eager_us = e0.elapsed_time(e1) * 1e3 / reps
            # the same launches recorded once and replayed, as the decode step above is timed: the figure reported
            g = capture(lambda: [moe_step() for _ in range(reps)])
            graph_us = float(np.median([timed_replay(g) for _ in range(3)])) * 1e3 / reps
            return graph_us, offsets, eager_us

        NTOK = 64
        rows = NTOK * TOPK
        moe_us, offsets, moe_eager_us = moe_leg(NTOK, args.moe_tile_only)
        small_us, small_offsets, small_eager_us = moe_leg(32)
        one_us, one_offsets, one_eager_us = moe_leg(1)
        moe_bytes = 3 * E * stride
        moe_ops = 2 * rows * 3 * F * H
        moe_out = {"workload": "IQ4_XS, 8 experts x (gate, up 14336x4096; down 4096x14336), 64 tokens, top-2 "
                               "(seeded fp32 router), pairs grouped per expert on the device"
                               + (" [--moe-tile-only: grouped matmuls on the tile kernel alone]" if args.moe_tile_only else ""),
                   "pairs": rows, "rows_per_expert": np.diff(offsets).tolist(), "us_per_step": round(moe_us, 1),
                   "us_per_step_launched_eagerly": round(moe_eager_us, 1),
                   "weight_bytes": moe_bytes, "weight_GBps": round(moe_bytes / moe_us / 1e3, 1),
                   "frac_hbm_peak": round(moe_bytes / moe_us / 1e3 / HBM_PEAK_GBPS, 4),
                   "int8_TOPS": round(moe_ops / moe_us / 1e6, 1),
                   "timed": "six layers in a replayed HIP graph (median of three replays); the whole layer: router + softmax + top-2 + grouping, gather + quantize, 3 grouped int8-MFMA "
                            "matmuls, SwiGLU + quantize, weighted combine (the 749 MB of expert weights exceed the "
                            "256 MB Infinity Cache, so every step streams them from HBM)"}
        moe_small = {"workload": "the same layer for a decode batch of 32 tokens (64 pairs): with a mean of 8 rows per "
                                 "expert the grouped matmuls take the few-token kernel (16 x 16 x 32 MFMA tiles)",
                     "rows_per_expert": np.diff(small_offsets).tolist(), "us_per_step": round(small_us, 1),
                     "us_per_step_launched_eagerly": round(small_eager_us, 1),
                     "weight_GBps": round(moe_bytes / small_us / 1e3, 1),
                     "frac_hbm_peak": round(moe_bytes / small_us / 1e3 / HBM_PEAK_GBPS, 4)}
        live = int((np.diff(one_offsets) > 0).sum())
        moe_one = {"workload": "the same layer for ONE token (MoeFfn::forward's own call: top-2, two expert rows): every "
                               "projection is one GEMV launch over the two chosen experts' matrices",
                   "us_per_step": round(one_us, 1), "us_per_step_launched_eagerly": round(one_eager_us, 1),
                   "experts_read": live, "weight_bytes": 3 * live * stride,
                   "weight_GBps": round(3 * live * stride / one_us / 1e3, 1),
                   "frac_hbm_peak": round(3 * live * stride / one_us / 1e3 / HBM_PEAK_GBPS, 4)}
        del wg, wu, wd

    # ---- CPU baseline: the reference's fused rows restated in C, same layer -------------
    cpu = None
    parity = None
    if not args.no_cpu_baseline:
        sys.path.insert(0, os.path.join(ROOT, "tests"))
        import oracle as O
        O.load()
        host_cores = os.cpu_count() or 1
        cores = min(host_cores, 16)  # threads actually used (the GPU box's CPU share)
        hw = {"q": layers[0]["q"].cpu().numpy(), "gate": layers[0]["gate"].cpu().numpy(),
              "up": layers[0]["up"].cpu().numpy(), "down": layers[0]["down"].cpu().numpy()}
        hx = x.cpu().numpy()

        avx2 = O.load_avx2() is not None

        def fused(t, w, a, n_rows, n_cols, threads):
            if avx2:
                return O.avx2_matvec_q8_fused(t, w, a, n_rows, n_cols, threads)
            return O.matvec_q8_fused_mt(t, w, a, n_rows, n_cols, threads)

        def cpu_step(threads):
            a = O.quantize_q8_0(hx)
            fused(O.Q8_0, hw["q"], a, H, H, threads)
            hg = fused(O.Q4_K, hw["gate"], a, F, H, threads)
            hu = fused(O.Q4_K, hw["up"], a, F, H, threads)
            b = O.quantize_q8_0(O.swiglu(hg, hu))
            fused(O.Q6_K, hw["down"], b, H, F, threads)

        def time_cpu(threads, budget_s):
            cpu_step(threads)
            n, t_begin = 0, time.perf_counter()
            while True:
                cpu_step(threads)
                n += 1
                el = time.perf_counter() - t_begin
                if el > budget_s or n >= 50:
                    return el / n, n

        # Parity gate beside the timing: the timed step once more on layer 0, each stage against the
        # oracle on the device's own input to that stage (activation bytes ==, fp32 within 1e-5 * |y|_inf).
        with torch.cuda.stream(stream):
            step(0)
            stream.synchronize()
        g_xq, g_hq = xq.cpu().numpy(), hq.cpu().numpy()
        g_y = {"q": yq.cpu().numpy(), "gate": yg.cpu().numpy(), "up": yu.cpu().numpy(), "down": yd.cpu().numpy()}

        def rel_err(got, want):
            return float(np.abs(got.astype(np.float64) - want).max() / max(float(np.abs(want).max()), 1e-30))

        if args.fused_quantize:
            parity = None  # this variant keeps no Q8_0 buffers to compare stage by stage
        else:
            a_ref = O.quantize_q8_0(hx)
            g_ref = O.matvec_q8_fused_mt(O.Q4_K, hw["gate"], g_xq, F, H, cores)
            u_ref = O.matvec_q8_fused_mt(O.Q4_K, hw["up"], g_xq, F, H, cores)
            errs = {"q_proj": rel_err(g_y["q"], O.matvec_q8_fused_mt(O.Q8_0, hw["q"], g_xq, H, H, cores)),
                    "ffn_down": rel_err(g_y["down"], O.matvec_q8_fused_mt(O.Q6_K, hw["down"], g_hq, H, F, cores))}
            if args.unfused_swiglu:
                errs["ffn_gate"], errs["ffn_up"] = rel_err(g_y["gate"], g_ref), rel_err(g_y["up"], u_ref)
                h_ref = O.quantize_q8_0(O.swiglu(g_y["gate"], g_y["up"]))
            else:  # the fused launch keeps gate / up in registers: compare h = silu(gate) * up instead
                h_f32 = torch.empty(F, dtype=torch.float32, device=dev)
                hq2 = torch.empty_like(hq)
                with torch.cuda.stream(stream):
                    linear.gate_up_swiglu_dev(Q4_K, layers[0]["gate"], layers[0]["up"], xq, h_f32, hq2, F, H)
                    stream.synchronize()
                g_h = h_f32.cpu().numpy()
                errs["ffn_gate_up_swiglu_h"] = rel_err(g_h, O.swiglu(g_ref, u_ref))
                h_ref = O.quantize_q8_0(g_h)
                assert np.array_equal(hq2.cpu().numpy(), g_hq)
            parity = {"acts_q8_bytes_equal": bool(np.array_equal(g_xq, a_ref)),
                      "h_q8_bytes_equal_fraction": round(float(np.mean(g_hq == h_ref)), 6),
                      "fp32_max_err_over_ymax": {k: float(f"{v:.3e}") for k, v in errs.items()},
                      "tolerance": 1e-5,
                      "pass": bool(np.array_equal(g_xq, a_ref) and max(errs.values()) <= 1e-5),
                      "checked_against": "scalar C restatement of the reference's fused rows, layer 0 of the timed step"}
            if not parity["pass"]:
                print("bench.py: PARITY GATE FAILED: " + json.dumps(parity), file=sys.stderr, flush=True)

        if args.f32_route:
            # the reference's other method on the CPU: gemv on unquantized fp32 activations, one call of ffn_gate,
            # beside the GPU's f32_route_* legs.  Where the host has AVX-512F: the intrinsics twin of the reference's
            # AVX-512 row (Q/simd/avx512/q4_k.rs:279-415) on `cores` threads, best of a few calls; else the scalar
            # restatement (Q/reference/q4_k.rs:135-178) on one thread.
            if O.load_avx512() is not None:
                O.avx512_gemv_q4_k(hw["gate"], hx, F, H, threads=cores)
                el, reps = 1e9, 0
                t_stop = time.perf_counter() + 3.0
                while time.perf_counter() < t_stop:
                    t_begin = time.perf_counter()
                    O.avx512_gemv_q4_k(hw["gate"], hx, F, H, threads=cores)
                    el = min(el, time.perf_counter() - t_begin)
                    reps += 1
                used, what = cores, f"AVX-512 twin of the reference's gemv row, {cores} threads (static row split), best of {reps} calls (the 33 MB matrix stays in the host's caches between them)"
            else:
                t_begin = time.perf_counter()
                O.gemv(O.Q4_K, hw["gate"], F, H, hx)
                el = time.perf_counter() - t_begin
                used, what = 1, "scalar C restatement on one host thread, one call"
            kernels["f32_route_cpu_q4k_gate_14336x4096"] = {
                "us_per_call": round(el * 1e6, 1), "launches": 1, "distinct_weight_sets": 1,
                "weight_GBps": round(F * row_bytes(Q4_K, H) / el / 1e9, 3), "frac_hbm_peak": None, "cores": used,
                "kind": "port", "sample": "gemv of ffn_gate 14336x4096 on fp32 activations: " + what}
        s_mt, n_mt = time_cpu(cores, 8.0)
        s_1t, n_1t = time_cpu(1, 8.0)
        cpu = {"value": round(step_weight_bytes / s_mt / 1e9, 3), "unit": "GB/s", "cores": cores, "host_cores": host_cores,
               "kind": "port",
               "sample_short": f"one layer of the timed step, {n_mt} repeats, {cores} threads (static row split); " +
                               ("AVX2 twin of the reference's fused rows" if avx2 else "scalar C restatement"),
               "sample": f"one layer (same 4 matrices, quantization of x, SwiGLU + quantization of h), {n_mt} repeats, static row split over "
                         f"{cores} threads; " + ("AVX2 intrinsics twin of the reference's fused rows (Q6_K body is scalar "
                         "there too)" if avx2 else "scalar C restatement of the reference's AVX2-tier fused rows"),
               "ms_per_step": round(s_mt * 1e3, 3),
               "single_thread": {"value": round(step_weight_bytes / s_1t / 1e9, 3), "ms_per_step": round(s_1t * 1e3, 3),
                                 "repeats": n_1t}}

    detail = {"timing": timing, "roofline": roofline, "cpu_baseline": cpu, "parity": parity, "kernels": kernels,
              "prefill": prefill, "moe": moe_out, "moe_32_tokens": moe_small, "moe_1_token": moe_one,
              "device": {"name": info["name"], "arch": info["arch"], "compute_units": info["compute_units"],
                         "clock_mhz": info["clock_khz"] / 1000.0, "weight_generation_s": round(gen_s, 1)}}
    if args.detail:
        with open(args.detail, "w") as f:
            json.dump(detail, f, indent=1)

    def short(k):  # per-kernel legs: time and fraction of the 8 TB/s peak (algorithmic bytes where the leg has them)
        return {"us": k["us_per_call"], "frac": k["frac_hbm_peak"]}

    def get(d, *path):
        for p in path:
            if d is None:
                return None
            d = d.get(p)
        return d

    launch_words = ("quantize x, q_proj, gate+up+SwiGLU+quantize (one launch), down" if not (args.fused_quantize or args.unfused_swiglu)
                    else "quantize x, q_proj, gate+up (one launch), SwiGLU+quantize, down" if not args.fused_quantize
                    else "q_proj, gate+up (one launch), SwiGLU, down, each quantizing its fp32 input itself")
    # where the targets of this path stand, in one flat object (fractions of the 8 TB/s HBM peak, of the 5 POPS int8 peak)
    targets = {"q4k_gate_up_swiglu_frac": pair_swiglu["frac_hbm_peak"], "q4k_gate_up_frac": pair["frac_hbm_peak"],
               "q4k_gate_frac": get(kernels, "q4k_gate_up_14336x4096", "frac_hbm_peak"),
               "q6k_down_frac": get(kernels, "q6k_down_4096x14336", "frac_hbm_peak"),
               "q8_0_q_proj_frac": get(kernels, "q8_0_q_proj_4096x4096", "frac_hbm_peak"),
               "c1_q4_0_frac": get(kernels, "c1_q4_0_4096x4096", "frac_hbm_peak"),
               "c3_lm_head_frac": get(kernels, "c3_lm_head_q6k_128256x4096", "frac_hbm_peak"),
               "c3_lm_head_us": get(kernels, "c3_lm_head_q6k_128256x4096", "us_per_call"),
               "c3_lm_head_top40_us": get(kernels, "c3_lm_head_then_candidates", "top40_three_launches_us"),
               "c3_lm_head_argmax_us": get(kernels, "c3_lm_head_then_candidates", "argmax_one_launch_us"),
               "prefill_frac_int8_peak": get(prefill, "frac_int8_peak"), "prefill_gemm_us": get(prefill, "gemm_us"),
               "prefill_TOPS": get(prefill, "TOPS"), "moe_us": get(moe_out, "us_per_step"),
               "moe_frac": get(moe_out, "frac_hbm_peak"),
               "batch16_q4k_4096x14336_us": get(kernels, "batch16_q4k_down_shape_4096x14336", "us_per_call"),
               "batch16_q6k_4096x14336_us": get(kernels, "batch16_q6k_down_4096x14336", "us_per_call")}
    out = {
        "metric": "Q4_K GEMV weight GB/s (% HBM peak); batch-512 prefill int8-MFMA TOPS",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 dot -> int32 group sums -> f32",
        "data": "synthetic",
        "config": {"workload": "Llama-3-8B decode projections, batch 1: q_proj 4096x4096 Q8_0, ffn_gate/ffn_up "
                               "14336x4096 Q4_K, ffn_down 4096x14336 Q6_K, Q8_0 activations",
                   "weight_bytes_per_step": step_weight_bytes, "distinct_layers": L,
                   "frac_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
                   "launch": "one HIP graph of all timed steps; per step " + launch_words,
                   "timing": {"replays": R, "reported": "median wall time of the replays / steps",
                              "ms_min": timing["ms_per_step_min"], "ms_max": timing["ms_per_step_max"],
                              "ms_hip_events": timing["ms_per_step_hip_events_median"]},
                   "targets": targets},
        "roofline": {"bound": "hbm", "kernel": dom_launch, "achieved": roofline["achieved"], "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": roofline["frac"], "traffic": roofline["traffic"],
                     "us_per_call": roofline["us_per_call"], "algorithmic_bytes": roofline["algorithmic_bytes"],
                     "others": {k: short(v) for k, v in kernels.items() if "frac_hbm_peak" in v}},
        "cpu_baseline": None if cpu is None else {
            "value": cpu["value"], "unit": "GB/s", "cores": cpu["cores"], "kind": "port",
            "sample": "",
            "ms_per_step": cpu["ms_per_step"], "single_thread_value": cpu["single_thread"]["value"]},
        "parity": None if parity is None else {
            "pass": parity["pass"], "acts_q8_bytes_equal": parity["acts_q8_bytes_equal"],
            "h_q8_bytes_equal_fraction": parity["h_q8_bytes_equal_fraction"],
            "fp32_max_err_over_ymax": parity["fp32_max_err_over_ymax"], "tolerance": 1e-5},
        "prefill": None if prefill is None else {
            "gemm_us": prefill["gemm_us"], "quantize_us": prefill["quantize_us"], "TOPS": prefill["TOPS"],
            "frac_int8_peak": prefill["frac_int8_peak"], "kernel": prefill["launch"].split(" ")[0],
            "int8_tile_kernel_gemm_us": prefill["int8_tile_kernel_gemm_us"], "mfma_only_TOPS": prefill["mfma_only_TOPS"],
            "other_formats_gemm_us": {k: v["gemm_us"] for k, v in prefill["same_shape_other_formats"].items()}},
        "moe": None if moe_out is None else {
            "us_64_tokens": moe_out["us_per_step"], "frac_64_tokens": moe_out["frac_hbm_peak"],
            "rows_per_expert": moe_out["rows_per_expert"], "us_32_tokens": moe_small["us_per_step"],
            "frac_32_tokens": moe_small["frac_hbm_peak"], "us_1_token": moe_one["us_per_step"],
            "frac_1_token": moe_one["frac_hbm_peak"]},
        "batch16": {k: {"us": v["us_per_call"], "tile_kernel_us": v["tile_kernel_us_per_call"]}
                    for k, v in kernels.items() if "tile_kernel_us_per_call" in v},
        "device": {"name": info["name"], "compute_units": info["compute_units"]},
    }
    if cpu is not None:
        out["cpu_baseline"]["sample"] = cpu["sample_short"]
    print(json.dumps(out), flush=True)
    if parity is not None and not parity["pass"]:
        sys.exit(3)  # the line above is still printed; a fast kernel with wrong results is not a result


if __name__ == "__main__":
    main()
