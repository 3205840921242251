#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-sweep]

One "step" = one decode-step call (M=1 token) of the benchmark's configuration 3 up/gate
layer (Llama-3-8B MLP, N=14336, K=4096, vector length 8, 65536-entry fp16
codebook, 16-bit indices, bf16 activations) on synthetic seeded data already
resident in HBM, through the kernel NPVQLinear uses for it: the slice-list
decode GEMV (one launch per call).  K steps are recorded into one HIP graph over a
rotating pool of weight/activation buffers larger than L2 + Infinity Cache and
timed with HIP events on the launch stream (median of 5 replays, caches flushed
before each), so `value` is kernel throughput, not Python launch overhead, and
the index stream really comes from HBM; `python_overhead_us` is what an eager
call adds on top.

Prints ONE JSON line: the headline value (algorithmic GB/s of the M=1 GEMV),
`roofline` for that kernel, `roofline_m384` for the tile GEMM, `footprint`,
`cpu_baseline` / `cpu_baselines` (the reference's CPU path restated with torch
ops, timed on this host, decode and matmul apart), and a `sweep` over the other
bands / configs (us per call, GB/s, TFLOP/s, fraction of peak).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0      # dense bf16 / fp16
METRIC = "VQ-linear µs/call + HBM GB/s (M=1), TFLOP/s (M=384), Llama-3-8B shapes"
POOL_BYTES = 640 << 20         # rotate through more than L2 (32 MB) + Infinity Cache (256 MB)
# HBM bytes per dispatch from rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE, scaled by what the same
# counters read for a plain copy of known size).  Not measured in this run: the profile summary named
# in `source` holds the command, the raw counter values and the date they were taken.
TRAFFIC = {
    "sliced_m1": {"bytes": 13577 * 1024 * 2 + 1932 * 1024, "source": "profiles/vq_sliced_gemv_cfg3_14336x4096_m1.md"},
    "tile_m384": {"bytes": 35573 * 1024 * 2 + 51082 * 1024, "source": "profiles/vq_tile_gemm_cfg3_14336x4096_m384.md"},
}
FLUSH_BYTES = 512 << 20        # written before every timed replay: nothing a replay reads is still cached


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sweep", action="store_true", help="headline kernel only")
    ap.add_argument("--case", default="", choices=["", "sliced_m1", "gemv_m1", "gemv_nc4096_m1", "gemv_cfg2_gateup_m1", "gemv_cfg2_down_m1", "tile_m256", "tile_m384", "tile_nc4096_m128", "dequant", "q4_gemv_m1", "q4_gemv_m16", "q4_gemv_4096_m16", "q4_gemv_28672_m1", "q4_tile_m128", "q4_tile_m256", "q4_tile_m512", "rvq_gemv_m1", "rvq_tile_m128",
                                                    "rms_norm_m4096", "vq_embedding_m4096", "q4_embedding_m4096"],
                    help="profiling aid: launch only this kernel `--steps` times (eagerly, one kernel per launch) "
                         "on the config-3 / config-5 shape (rvq_*: the config-4 4096x4096 projection) and print a one-line JSON with its HIP-event time")
    ap.add_argument("--ceilings", action="store_true",
                    help="measure only the memory-system ceilings for config 3's access pattern: plain read of "
                         "the index stream, and one 16-byte table lookup per index for several table sizes")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a plain device copy of 256 MiB (10 launches): the known-size kernel "
                         "the FETCH_SIZE / WRITE_SIZE counters are scaled against")
    return ap.parse_args()


def gen(seed):
    return torch.Generator().manual_seed(seed)


def time_graph(fn, n_rot, steps, warmup, dev, replays=5, flush=None):
    """Median microseconds per call of fn(i) over `replays` replays of one HIP graph of `steps` calls.

    Events are recorded on the stream the graph is launched on (torch's current
    stream), before and after each replay.  `flush`, when given, runs before every
    replay, outside the timed bracket: it overwrites a buffer larger than L2 +
    Infinity Cache, so that no replay finds its weights cached by the one before.
    """
    for i in range(max(warmup, 1)):
        fn(i % n_rot)
    torch.cuda.synchronize(dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(steps):
            fn(i % n_rot)
    graph.replay()  # untimed: first replay uploads the graph
    torch.cuda.synchronize(dev)
    times = []
    for _ in range(replays):
        if flush is not None:
            flush()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize(dev)
        times.append(e0.elapsed_time(e1) * 1e3 / steps)
    return sorted(times)[len(times) // 2]


def host_cpu_description():
    """Model string of the host CPU with what /proc/cpuinfo adds to it (family / model / stepping, logical CPUs,
    sockets): the name alone can be as short as "AMD EPYC" on virtualised hosts."""
    fields, logical, sockets = {}, 0, set()
    try:
        with open("/proc/cpuinfo") as fh:
            for ln in fh:
                key, _, val = ln.partition(":")
                key, val = key.strip(), val.strip()
                if key == "processor":
                    logical += 1
                elif key == "physical id":
                    sockets.add(val)
                elif key in ("model name", "cpu family", "model", "stepping", "vendor_id") and key not in fields:
                    fields[key] = val
    except OSError:
        return ""
    name = fields.get("model name", fields.get("vendor_id", "unknown"))
    return (f"{name} (family {fields.get('cpu family', '?')} model {fields.get('model', '?')} stepping "
            f"{fields.get('stepping', '?')}; {logical} logical CPUs visible, {max(len(sockets), 1)} socket(s))")


def rot_for(bytes_per_buffer, cap=512):
    """Buffers in a rotating pool: enough for POOL_BYTES, at most `cap` (small layers)."""
    return max(2, min(cap, -(-POOL_BYTES // max(int(bytes_per_buffer), 1))))


def time_eager(fn, n_rot, calls, dev):
    """(host, wall) microseconds per call when every call is issued from Python: `host` is the time the
    interpreter spends issuing one call (argument checks, ctypes, the HIP launch; the GPU runs behind),
    `wall` includes waiting for the last call to finish."""
    for i in range(10):
        fn(i % n_rot)
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for i in range(calls):
        fn(i % n_rot)
    t1 = time.perf_counter()
    torch.cuda.synchronize(dev)
    return (t1 - t0) * 1e6 / calls, (time.perf_counter() - t0) * 1e6 / calls


def vq_case(dev, seed, n, k, nc, bits, act, n_rot):
    from neuropress_amd.transforms.vq_packing import IndexPacking

    g = gen(seed)
    cb = (torch.randn(nc, 8, generator=g) * 0.02).to(torch.float16)
    n_idx = n * (k // 8)
    if bits == 16:
        base = torch.randint(0, nc, (n_idx,), generator=g, dtype=torch.int32).to(torch.int16).view(torch.uint8)
    else:
        base = IndexPacking.pack(torch.randint(0, nc, (n_idx,), generator=g), bits)
    x = torch.randn(16, k, generator=g).to(act)
    d_base = base.to(dev)
    pool = [d_base] + [d_base.clone() for _ in range(n_rot - 1)]
    return dict(cb=cb, packed=base, x=x, d_cb=cb.to(dev), d_cb_act=cb.to(act).to(dev), pool=pool,
                n=n, k=k, nc=nc, bits=bits, act=act, idx_bytes=base.numel())


def vq_alg_bytes(c, m):
    return c["idx_bytes"] + c["nc"] * 16 + m * c["k"] * 2 + m * c["n"] * 2


def check_against_cpu(y_gpu, y_cpu):
    err = (y_gpu.float().cpu() - y_cpu.float()).abs()
    bound = 1e-2 + 1e-2 * y_cpu.float().abs()
    return bool((err <= bound).all()), float(err.max())


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: the path has no multi-GPU component (got --gpus {args.gpus}). "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (torch.cuda.is_available() is False).", file=sys.stderr)
        sys.exit(2)
    from neuropress_amd import _lib, kernels

    _lib.load()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibrate_copy:
        nbytes = 256 << 20
        src = torch.empty(nbytes // 4, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize(dev)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize(dev)
        print(json.dumps({"calibration": "device copy", "bytes_read": nbytes, "bytes_written": nbytes, "launches": 10}))
        return

    if args.case:
        from neuropress_amd.t2n.packing import BitPacking4
        from neuropress_amd.transforms.vq_packing import IndexPacking

        n, k = 14336, 4096
        g = gen(1003)
        n_rot = 48  # 48 x 14.7 MB index streams: more than L2 + Infinity Cache
        if args.case in ("rms_norm_m4096", "vq_embedding_m4096", "q4_embedding_m4096"):
            m, hdim, vocab, flops = 4096, 4096, 128256, 0.0
            if args.case == "rms_norm_m4096":
                wn = (torch.rand(hdim, generator=g) + 0.5).to(torch.bfloat16).to(dev)
                pool = [torch.randn(m, hdim, generator=g).to(torch.bfloat16).to(dev) for _ in range(n_rot)]
                fn = lambda i: kernels.rms_norm(pool[i], wn, 1e-6)
                alg = 2 * m * hdim * 2 + hdim * 2
            else:
                pool = [torch.randint(0, vocab, (m,), generator=g).to(dev) for _ in range(n_rot)]
                if args.case == "vq_embedding_m4096":
                    cbe = (torch.randn(65536, 8, generator=g) * 0.02).to(torch.float16).to(dev)
                    tab = torch.randint(0, 65536, (vocab, hdim // 8), generator=g, dtype=torch.int32).to(torch.int16).to(dev)
                    fn = lambda i: kernels.vq_embedding(pool[i], tab, cbe, 64.0, None, torch.bfloat16)
                    alg = m * (8 + hdim // 8 * 2 + hdim // 8 * 16 + hdim * 2)
                else:
                    qblob = torch.randint(0, 256, (vocab, hdim // 2), generator=g, dtype=torch.int32).to(torch.uint8).to(dev)
                    qsc = (torch.rand(vocab * hdim // 32, generator=g) * 0.019 + 0.001).to(torch.float16).to(dev)
                    fn = lambda i: kernels.q_embedding(pool[i], qblob, qsc, 4, 32, None, None, 64.0, torch.bfloat16)
                    alg = m * (8 + hdim // 2 + hdim // 32 * 2 + hdim * 2)
        elif args.case.startswith("rvq"):
            # config 4 q/o projection: residual VQ, Zipf(1.1) indices, per-row scale and bias, fp16
            n, k = 4096, 4096
            g, cnt = gen(1004), n * k // 8
            pz = 1.0 / torch.arange(1, 65537, dtype=torch.float64) ** 1.1
            cbm = (torch.randn(65536, 8, generator=g) * 0.02).to(torch.float16).to(dev)
            cbr = (torch.randn(256, 8, generator=g) * 0.02).to(torch.float16).to(dev)
            pm = torch.multinomial(pz / pz.sum(), cnt, replacement=True, generator=g).to(torch.int32).to(torch.int16).view(torch.uint8)
            pr = torch.multinomial(pz[:256] / pz[:256].sum(), cnt, replacement=True, generator=g).to(torch.uint8)
            rsc = (torch.rand(n, generator=g) + 0.5).to(torch.float16).to(dev)
            rbi = (torch.randn(n, generator=g) * 0.01).to(torch.float16).to(dev)
            n_rot = 32
            pool = [(pm.to(dev).clone(), pr.to(dev).clone()) for _ in range(n_rot)]
            m = 1 if args.case == "rvq_gemv_m1" else 128
            x = torch.randn(m, k, generator=g).to(torch.float16).to(dev)
            fn = lambda i: kernels.rvq_linear(x, pool[i][0], 16, pool[i][1], 8, cbm, cbr, rsc, rbi, n, tile=(m > 32))
            alg, flops = cnt * 3 + (65536 + 256) * 16 + n * 4 + m * k * 2 + m * n * 2, 2.0 * m * n * k
        elif args.case.startswith("q4"):
            if args.case == "q4_gemv_28672_m1":  # twice the rows: the resident-grid int4 GEMV takes it
                n, n_rot = 28672, 16
            if args.case == "q4_gemv_4096_m16":  # config 5's square layer: one row tile per workgroup
                n, n_rot = 4096, 96
            blob = BitPacking4.compress(torch.randint(0, 16, (n, k), generator=g, dtype=torch.int64).to(torch.uint8))
            sc = (torch.rand(n * k // 32, generator=g) * 0.019 + 0.001).to(torch.float16).to(dev)
            pool = [blob.to(dev).clone() for _ in range(n_rot)]
            m = {"q4_gemv_m1": 1, "q4_gemv_28672_m1": 1, "q4_gemv_m16": 16, "q4_gemv_4096_m16": 16, "q4_tile_m256": 256, "q4_tile_m512": 512}.get(args.case, 128)
            x = torch.randn(m, k, generator=g).to(torch.float16).to(dev)
            fn = lambda i: kernels.q_linear(x, pool[i], sc, 4, 32)
            alg, flops = n * k // 2 + n * k // 32 * 2 + m * k * 2 + m * n * 2, 2.0 * m * n * k
        else:
            nc, bits = (4096, 12) if args.case in ("gemv_nc4096_m1", "tile_nc4096_m128") else (65536, 16)
            if args.case.startswith("gemv_cfg2"):  # config 2's own layers: 4096-row codebook, int16 stream
                n, k = (8192, 2048) if args.case == "gemv_cfg2_gateup_m1" else (2048, 8192)
                nc, bits, n_rot = 4096, 16, 160
            cb = (torch.randn(nc, 8, generator=g) * 0.02).to(torch.float16)
            if bits == 16:
                base = torch.randint(0, nc, (n * k // 8,), generator=g, dtype=torch.int32).to(torch.int16).view(torch.uint8)
            else:
                base = IndexPacking.pack(torch.randint(0, nc, (n * k // 8,), generator=g), bits)
            pool = [base.to(dev).clone() for _ in range(n_rot)]
            cb16, cbb = cb.to(dev), cb.to(torch.bfloat16).to(dev)
            m = 256 if args.case == "tile_m256" else 384 if args.case == "tile_m384" else 128 if args.case == "tile_nc4096_m128" else 1
            x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(dev)
            if args.case.startswith("gemv_cfg2"):
                x, cbb = x.to(torch.float16), cb16  # config 2 runs in fp16
            if args.case == "sliced_m1":
                sl0 = kernels.vq_slice_indices(base, bits, n, k, 8, nc, device=dev)
                n_rot = rot_for(sl0.total_bytes)  # more than L2 + Infinity Cache, as in the main run
                spool = [sl0] + [kernels.SlicedIndices(sl0.blob.clone(), sl0.header) for _ in range(n_rot - 1)]
                ws = torch.zeros(sl0.workspace_bytes(1) // 4, device=dev, dtype=torch.float32)
                fn = lambda i: kernels.vq_linear_sliced(x, spool[i], cbb, None, workspace=ws)
            elif args.case in ("tile_m256", "tile_m384", "tile_nc4096_m128"):
                fn = lambda i: kernels.vq_gemm_tile(x, pool[i], cbb, bits, n, None)
            elif args.case == "dequant":
                fn = lambda i: kernels.vq_dequant(pool[i], cb16, bits, n, k, torch.bfloat16)
            else:
                fn = lambda i: kernels.vq_linear(x, pool[i], cbb, bits, 8, None, n)
            alg = base.numel() + nc * 16 + m * k * 2 + m * n * 2 + (n * k * 2 if args.case == "dequant" else 0)
            flops = 2.0 * m * n * k
        for i in range(args.warmup):
            fn(i % n_rot)
        torch.cuda.synchronize(dev)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(args.steps):
            fn(i % n_rot)
        e1.record()
        torch.cuda.synchronize(dev)
        us = e0.elapsed_time(e1) * 1e3 / args.steps
        print(json.dumps({"case": args.case, "steps": args.steps, "us_per_launch_incl_python": round(us, 2),
                          "algorithmic_bytes": alg, "flops": flops}))
        return

    if args.ceilings:
        n_idx = 14336 * 512
        n_rot = max(2, POOL_BYTES // (n_idx * 2))
        g = gen(1003)
        base = torch.randint(0, 65536, (n_idx,), generator=g, dtype=torch.int32).to(torch.int16).to(dev)
        pool = [base] + [base.clone() for _ in range(n_rot - 1)]
        table = (torch.randn(65536, 8, generator=g) * 0.02).to(torch.bfloat16).to(dev)
        sink = torch.zeros(16, dtype=torch.uint8, device=dev)
        st = lambda: torch.cuda.current_stream(dev).cuda_stream
        out = {"ceilings": "config 3 access pattern, 7 340 032 16-bit indices (14.7 MB), rotating pool",
               "stream_read_us": round(time_graph(lambda i: _lib.call(
                   "npamd_diag_stream_read", pool[i].data_ptr(), n_idx * 2, sink.data_ptr(), st()),
                   n_rot, args.steps, args.warmup, dev), 2)}
        for entries in (256, 2048, 4096, 16384, 65536):
            out[f"gather_global_{entries}_rows_us"] = round(time_graph(lambda i: _lib.call(
                "npamd_diag_gather", pool[i].data_ptr(), n_idx, table.data_ptr(), entries, 0, sink.data_ptr(), st()),
                n_rot, args.steps, args.warmup, dev), 2)
        for entries in (256, 4096, 8192):
            out[f"gather_lds_{entries}_rows_us"] = round(time_graph(lambda i: _lib.call(
                "npamd_diag_gather", pool[i].data_ptr(), n_idx, table.data_ptr(), entries, 1, sink.data_ptr(), st()),
                n_rot, args.steps, args.warmup, dev), 2)
        print(json.dumps(out))
        return

    # Buffer read before every timed replay (outside the event bracket): larger than L2 (32 MB) +
    # Infinity Cache (256 MB), so a replay never finds its weights cached by the previous one.  It is read,
    # not written: dirty lines would be written back during the replay that follows.  Within a replay every
    # row below visits each buffer of its rotating pool once (or, for the headline, wraps only after the
    # pool's 640 MB), so what is timed does not depend on --steps.
    flush_buf = torch.zeros(FLUSH_BYTES // 4, dtype=torch.float32, device=dev)

    def flush():
        flush_buf.sum()

    def timed(fn, n_rot, steps=None, warmup=3):
        return time_graph(fn, n_rot, n_rot if steps is None else steps, warmup, dev, flush=flush)

    # ---------------- headline: config 3 up/gate, M = 1 --------------------------
    n, k = 14336, 4096
    n_rot = rot_for(n * k // 8 * 2)
    c3 = vq_case(dev, 1003, n, k, 65536, 16, torch.bfloat16, n_rot)
    xs = [torch.randn(1, k, generator=gen(7 + i)).to(torch.bfloat16).to(dev) for i in range(n_rot)]
    ys = [None] * n_rot
    sl0 = kernels.vq_slice_indices(c3["packed"], 16, n, k, 8, 65536, device=dev)
    s_rot = rot_for(sl0.total_bytes)
    spool = [sl0] + [kernels.SlicedIndices(sl0.blob.clone(), sl0.header) for _ in range(s_rot - 1)]
    ws = torch.zeros(sl0.workspace_bytes(1) // 4, device=dev, dtype=torch.float32)

    def step(i):
        ys[i % n_rot] = kernels.vq_linear_sliced(xs[i % n_rot], spool[i], c3["d_cb_act"], None, workspace=ws)

    us = time_graph(step, s_rot, args.steps, args.warmup, dev, flush=flush)
    alg = vq_alg_bytes(c3, 1)
    gbs = alg / us / 1e3
    host_us, wall_us = time_eager(step, s_rot, 200, dev)
    us_warm = time_graph(lambda i: step(0), 1, max(args.steps, 20), 2, dev)  # one blob, no flush: served by the Infinity Cache

    # correctness gate on the timed configuration (decode bit-exact, output within 1e-2 + 1e-2 |ref|)
    w_gpu = kernels.vq_dequant(c3["pool"][0], c3["d_cb"], 16, n, k, torch.bfloat16)
    idx = (c3["packed"].view(torch.int16).to(torch.int64) & 0xFFFF)
    decode_exact = bool(torch.equal(w_gpu.cpu(), c3["cb"][idx].reshape(n, k).to(torch.bfloat16)))
    y_ref = xs[0].float() @ w_gpu.float().T
    ok, max_abs = check_against_cpu(ys[0], y_ref.cpu())

    # the same call through the module, eagerly: what a caller that does not capture a graph pays per call
    from neuropress_amd.nn.np_vq_linear import NPVQLinear, VQProxy

    layer = NPVQLinear(VQProxy(c3["cb"]).to(dev), c3["packed"], 16, n, k, 8, "cuda_wmma").to(dev)
    has_lists = bool(layer.prepare_sliced())
    host_us_module, wall_us_module = time_eager(lambda i: layer(xs[i % n_rot]), n_rot, 200, dev)
    dense_bytes = n * k * 2
    footprint = {
        "layer": "config 3 up/gate 14336x4096",
        "packed_index_stream_bytes": int(c3["idx_bytes"]),
        "slice_list_bytes": int(sl0.total_bytes),
        "codebook_bytes_fp16_plus_bf16_copy": 2 * 65536 * 16,
        "resident_bytes_all_bands": int(c3["idx_bytes"] + sl0.total_bytes + 2 * 65536 * 16),
        "resident_bytes_decode_only": int(sl0.total_bytes + 65536 * 16),
        "dense_bf16_bytes": dense_bytes,
        "resident_over_dense_all_bands": round((c3["idx_bytes"] + sl0.total_bytes + 2 * 65536 * 16) / dense_bytes, 4),
        "resident_over_dense_decode_only": round((sl0.total_bytes + 65536 * 16) / dense_bytes, 4),
        "note": "the codebook (and its bf16 copy) is shared by every layer bound to the same VQProxy; "
                "the slice lists serve calls of 1-7 tokens, the packed stream every other band",
    }
    del layer
    torch.cuda.empty_cache()

    # The most any kernel could show on this shape, measured in this run: a plain read (one 16-byte load per
    # lane, nothing else) of as many bytes as the reference's format holds, launch included.
    sink = torch.zeros(16, dtype=torch.uint8, device=dev)
    read16 = alg // 16 * 16
    assert read16 <= sl0.total_bytes
    floor_us = time_graph(lambda i: _lib.call("npamd_diag_stream_read", spool[i].blob.data_ptr(), read16, sink.data_ptr(),
                                              torch.cuda.current_stream(dev).cuda_stream),
                          s_rot, s_rot, 3, dev, flush=flush)

    result = {
        "metric": METRIC,
        "value": round(gbs, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us / 1e3, 6),
        "us_per_call": round(us, 3),
        "cache_warm_us_per_call": round(us_warm, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic (seed 1003; uniform 16-bit indices, N(0,0.02) fp16 codebook, N(0,1) bf16 activations)",
        "timing": "HIP graph of the calls, HIP events on the launch stream, median of 5 replays, 512 MB cache "
                  "flush before each replay (outside the bracket), rotating weight pools of 640 MB",
        "config": {
            "workload": "BASELINE config 3: Llama-3-8B MLP up/gate 14336x4096, VL=8, 65536-entry fp16 codebook, "
                        "16-bit indices, bf16, M=1 (band a: slice-list decode GEMV, one kernel per call)",
            "N": n, "K": k, "M": 1, "rotating_pool_MB": round(s_rot * sl0.total_bytes / 2**20),
        },
        # host time to issue one eager call (Python + ctypes + HIP launch); a graph replay pays none of it
        "python_overhead_us": round(host_us, 2),
        "eager_us_per_call": {"kernels.vq_linear_sliced": {"host_issue": round(host_us, 2), "wall": round(wall_us, 2)},
                              "NPVQLinear.forward": {"host_issue": round(host_us_module, 2), "wall": round(wall_us_module, 2)},
                              "graph_replay": round(us, 3), "module_has_slice_lists": has_lists},
        "footprint": footprint,
    }
    # `roofline`, `roofline_m384`, `cpu_baseline` and `checks` are appended last, behind the long `sweep` and
    # `cpu_baselines` lists, so that a reader who keeps only the end of the line still has them.
    roofline = {
        "bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": round(gbs / HBM_PEAK_GBS, 4),
        "traffic": TRAFFIC["sliced_m1"]["bytes"], "traffic_source": TRAFFIC["sliced_m1"]["source"],
        "kernel": "sliced_gemv_kernel<bf16, M=1>", "algorithmic_bytes_per_launch": alg,
        "avg_launch_us": round(us, 3),
        # plain read of the same bytes in this run (launch included): what a kernel that only read them would take
        "floor_us": round(floor_us, 3), "frac_at_floor": round(alg / floor_us / 1e3 / HBM_PEAK_GBS, 4),
        "streamed_bytes_per_launch": int(sl0.total_bytes + sl0.n_workgroups * sl0.slice_rows * 16 + k * 2 + n * 2),
        "note": "achieved = bytes of the reference's format (index stream + codebook + x + y) / launch duration",
    }
    checks = {"decode_bit_exact": decode_exact, "output_within_1e-2": ok, "max_abs_err": max_abs}

    # The second half of the metric: the tile-decode GEMM at M = 384 on the same layer, priced against the
    # dense bf16 MFMA peak.  Timed here so that the line carries it with --no-sweep too.
    m2 = 384
    xm2 = [torch.randn(m2, k, generator=gen(60 + m2)).to(torch.bfloat16).to(dev) for _ in range(2)]
    us_tile = timed(lambda i: kernels.vq_gemm_tile(xm2[i % 2], c3["pool"][i], c3["d_cb_act"], 16, n, None), n_rot)
    flops2 = 2.0 * m2 * n * k
    y2 = kernels.vq_gemm_tile(xm2[0], c3["pool"][0], c3["d_cb_act"], 16, n, None)
    ok2, max_abs2 = check_against_cpu(y2, (xm2[0].float() @ w_gpu.float().T).cpu())
    # The matrix pipes alone, in this run: the same number of MFMA 32x32x16 spread over every compute unit,
    # random finite operands, nothing else in the kernel.
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    per_wave = -(-int(flops2 / (2 * 32 * 32 * 16)) // (cus * 4))
    ops = torch.randn(7 * 64 * 8, generator=gen(9)).to(torch.bfloat16).to(dev)
    us_mfma = time_graph(lambda i: _lib.call("npamd_diag_mfma", ops.data_ptr(), cus, per_wave, _lib.BF16, sink.data_ptr(),
                                             torch.cuda.current_stream(dev).cuda_stream), 1, 20, 3, dev)
    roofline_m384 = {
        "bound": "mfma", "achieved": round(flops2 / us_tile / 1e6, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": round(flops2 / us_tile / 1e6 / MFMA_PEAK_TFLOPS, 4),
        "traffic": TRAFFIC["tile_m384"]["bytes"], "traffic_source": TRAFFIC["tile_m384"]["source"],
        "kernel": "tile2_gemm_kernel<bf16, MW=3, VQ 16-bit> (128 columns, eight waves, K in two halves)", "flops_per_launch": flops2,
        "avg_launch_us": round(us_tile, 3), "M": m2, "output_within_1e-2": ok2, "max_abs_err": max_abs2,
        # the same flops as MFMAs only, on all compute units, in this run
        "floor_us": round(us_mfma, 3), "frac_at_floor": round(flops2 / us_mfma / 1e6 / MFMA_PEAK_TFLOPS, 4),
        "note": "same layer as `roofline`, 384 tokens; one launch decodes every weight once",
    }
    x384_cpu = xm2[0].cpu()
    del xm2, y2

    # ---------------- sweep over the other bands / configs ----------------------
    # Every row: the call timed as above, and the same call's output checked against the dense
    # product of the decoded weight in f32 (the decode kernels are bit-exact against the oracle,
    # tested): max abs error, its largest ratio to the bound 1e-2 + 1e-2 |ref|, and whether it holds.
    sweep = []
    if not args.no_sweep:
        def check(y, ref):
            err = (y.float() - ref).abs()
            bound = 1e-2 + 1e-2 * ref.abs()
            return {"max_abs_err": round(float(err.max()), 6), "err_over_bound": round(float((err / bound).max()), 3),
                    "ok": bool((err <= bound).all())}

        def run(name, band, m, f, rot, alg_bytes, flops, ref=None, steps=None, warm=3):
            us_ = timed(f, rot, steps, warm)
            row = {"case": name, "band": band, "M": m, "us": round(us_, 2),
                   "GBps": round(alg_bytes / us_ / 1e3, 1), "hbm_frac": round(alg_bytes / us_ / 1e3 / HBM_PEAK_GBS, 4),
                   "TFLOPs": round(flops / us_ / 1e6, 1), "mfma_frac": round(flops / us_ / 1e6 / MFMA_PEAK_TFLOPS, 4)}
            if ref is not None:
                row.update(check(f(0), ref()))
            sweep.append(row)

        def xpair(m, kk, seed, act):
            return [torch.randn(m, kk, generator=gen(seed + j)).to(act).to(dev) for j in range(2)]

        w32 = w_gpu.float()  # config 3 up/gate, decoded above and found bit-exact
        name = "cfg3 14336x4096 bf16"
        for m in (2, 4, 7):
            xm = xpair(m, k, 50 + m, torch.bfloat16)
            ws2 = torch.zeros(sl0.workspace_bytes(m) // 4, device=dev, dtype=torch.float32)
            run(name, "a:sliced-gemv", m,
                lambda i: kernels.vq_linear_sliced(xm[i % 2], spool[i], c3["d_cb_act"], None, workspace=ws2), s_rot,
                vq_alg_bytes(c3, m), 2.0 * m * n * k, ref=lambda: xm[0].float() @ w32.T)
        del spool[1:]
        torch.cuda.empty_cache()
        for m in (1, 2, 16, 32):  # 32: two 16-token tiles per decoded operand
            xm = xpair(m, k, 50 + m, torch.bfloat16)
            run(name, "a:fused-gemv", m, lambda i: kernels.vq_linear(xm[i % 2], c3["pool"][i], c3["d_cb_act"], 16, 8, None, n),
                n_rot, vq_alg_bytes(c3, m), 2.0 * m * n * k, ref=lambda: xm[0].float() @ w32.T)
        for m in (64, 384, 1024, 4096):
            xm = xpair(m, k, 60 + m, torch.bfloat16)
            steps_m = None if m <= 1024 else 12
            ref = lambda: xm[0].float() @ w32.T
            run(name, "b:tile-gemm", m, lambda i: kernels.vq_gemm_tile(xm[i % 2], c3["pool"][i], c3["d_cb_act"], 16, n, None),
                n_rot, vq_alg_bytes(c3, m), 2.0 * m * n * k, ref=ref, steps=steps_m, warm=2)
            run(name, "c:decode+gemm", m, lambda i: torch.nn.functional.linear(
                xm[i % 2], kernels.vq_dequant(c3["pool"][i], c3["d_cb"], 16, n, k, torch.bfloat16)),
                n_rot, vq_alg_bytes(c3, m), 2.0 * m * n * k, ref=ref, steps=steps_m, warm=2)
            del xm
        del c3["pool"][1:], w32
        torch.cuda.empty_cache()
        # config 3 down-proj shape
        name = "cfg3 4096x14336 bf16"
        c3d = vq_case(dev, 1003, 4096, 14336, 65536, 16, torch.bfloat16, n_rot)
        w32 = kernels.vq_dequant(c3d["pool"][0], c3d["d_cb"], 16, 4096, 14336, torch.bfloat16).float()
        sld = kernels.vq_slice_indices(c3d["packed"], 16, 4096, 14336, 8, 65536, device=dev)
        sdpool = [sld] + [kernels.SlicedIndices(sld.blob.clone(), sld.header) for _ in range(rot_for(sld.total_bytes) - 1)]
        for m in (1, 2):
            wsd = torch.zeros(sld.workspace_bytes(m) // 4, device=dev, dtype=torch.float32)
            xm = xpair(m, 14336, 70 + m, torch.bfloat16)
            run(name, "a:sliced-gemv", m,
                lambda i: kernels.vq_linear_sliced(xm[i % 2], sdpool[i], c3d["d_cb_act"], None, workspace=wsd), len(sdpool),
                vq_alg_bytes(c3d, m), 2.0 * m * 4096 * 14336, ref=lambda: xm[0].float() @ w32.T)
        del sdpool, sld
        torch.cuda.empty_cache()
        for m, band in ((1, "a:fused-gemv"), (16, "a:fused-gemv"), (64, "b:tile-gemm"), (384, "b:tile-gemm"),
                        (1024, "b:tile-gemm"), (4096, "b:tile-gemm")):
            xm = xpair(m, 14336, 70 + m, torch.bfloat16)
            if band == "a:fused-gemv":
                f = lambda i: kernels.vq_linear(xm[i % 2], c3d["pool"][i], c3d["d_cb_act"], 16, 8, None, 4096)
            else:
                f = lambda i: kernels.vq_gemm_tile(xm[i % 2], c3d["pool"][i], c3d["d_cb_act"], 16, 4096, None)
            run(name, band, m, f, n_rot, vq_alg_bytes(c3d, m), 2.0 * m * 4096 * 14336,
                ref=lambda: xm[0].float() @ w32.T, steps=None if m <= 1024 else 12, warm=2)
            del xm
        del c3d, w32
        torch.cuda.empty_cache()
        # config 2: 4096-entry codebook, fp16.  Every shape with the index stream as int16 (the bytes the
        # configuration is quoted on); gate/up also with the 12-bit stream and a column permutation.
        for label, nn_, kk in (("q/o", 2048, 2048), ("k/v", 512, 2048), ("gate/up", 8192, 2048), ("down", 2048, 8192)):
            rot = rot_for(nn_ * kk // 8 * 2)
            cc = vq_case(dev, 1002, nn_, kk, 4096, 16, torch.float16, rot)
            w32 = kernels.vq_dequant(cc["pool"][0], cc["d_cb"], 16, nn_, kk, torch.float16).float()
            for m in (1, 2):
                xm = xpair(m, kk, 80 + m, torch.float16)
                run(f"cfg2 {label} {nn_}x{kk} f16 int16 stream", "a:gemv", m,
                    lambda i: kernels.vq_linear(xm[i % 2], cc["pool"][i], cc["d_cb"], 16, 8, None, nn_), rot,
                    vq_alg_bytes(cc, m), 2.0 * m * nn_ * kk, ref=lambda: xm[0].float() @ w32.T)
            del cc, w32
            torch.cuda.empty_cache()
        for name, (nn_, kk, nc, bits), ms in (("cfg2 gate/up 8192x2048 f16 12-bit stream", (8192, 2048, 4096, 12), (1, 2, 32)),
                                              ("cfg1 2048x640 f16 8-bit", (2048, 640, 256, 8), (1, 16))):
            rot = rot_for(nn_ * kk // 8 * bits // 8)
            cc = vq_case(dev, 1002 if bits == 12 else 1001, nn_, kk, nc, bits, torch.float16, rot)
            w32 = kernels.vq_dequant(cc["pool"][0], cc["d_cb"], bits, nn_, kk, torch.float16).float()
            for m in ms:
                xm = xpair(m, kk, 80 + m, torch.float16)
                ref = lambda: xm[0].float() @ w32.T
                run(name, "a:gemv", m, lambda i: kernels.vq_linear(xm[i % 2], cc["pool"][i], cc["d_cb"], bits, 8, None, nn_),
                    rot, vq_alg_bytes(cc, m), 2.0 * m * nn_ * kk, ref=ref)
                if m == 1 and bits == 12:
                    # the same call with a column permutation: gathered inside the GEMV, or by torch in front of it
                    perm = torch.randperm(kk, generator=gen(90)).to(dev)
                    p32 = perm.to(torch.int32)
                    refp = lambda: xm[0][:, perm].float() @ w32.T
                    run(name + " column_perm", "a:gemv, gather fused", m,
                        lambda i: kernels.vq_linear(xm[i % 2], cc["pool"][i], cc["d_cb"], bits, 8, None, nn_, column_perm=p32),
                        rot, vq_alg_bytes(cc, m) + kk * 4, 2.0 * m * nn_ * kk, ref=refp)
                    run(name + " column_perm", "a:torch gather + gemv", m,
                        lambda i: kernels.vq_linear(xm[i % 2][:, perm], cc["pool"][i], cc["d_cb"], bits, 8, None, nn_),
                        rot, vq_alg_bytes(cc, m) + kk * 8, 2.0 * m * nn_ * kk, ref=refp)
            if bits == 12:
                # the same layer in the token bands the configuration itself does not list: tile GEMM with the
                # 4096-row codebook looked up in LDS, against decode + GEMM
                for m in (64, 256):
                    xm = xpair(m, kk, 80 + m, torch.float16)
                    ref = lambda: xm[0].float() @ w32.T
                    run(name, "b:tile-gemm", m, lambda i: kernels.vq_gemm_tile(xm[i % 2], cc["pool"][i], cc["d_cb"], bits, nn_, None),
                        rot, vq_alg_bytes(cc, m), 2.0 * m * nn_ * kk, ref=ref)
                    run(name, "c:decode+gemm", m, lambda i: torch.nn.functional.linear(
                        xm[i % 2], kernels.vq_dequant(cc["pool"][i], cc["d_cb"], bits, nn_, kk, torch.float16)),
                        rot, vq_alg_bytes(cc, m), 2.0 * m * nn_ * kk, ref=ref)
            del cc, w32
            torch.cuda.empty_cache()
        # config 4: residual VQ (65536 + 256 entry codebooks, Zipf(1.1) indices, per-row scale / bias), fp16
        def zipf(gq, nc, count):
            pz = 1.0 / torch.arange(1, nc + 1, dtype=torch.float64) ** 1.1
            return torch.multinomial(pz / pz.sum(), count, replacement=True, generator=gq)

        for nn_, kk in ((4096, 4096), (1024, 4096)):
            g = gen(1004)
            cnt = nn_ * kk // 8
            cbm = (torch.randn(65536, 8, generator=g) * 0.02).to(torch.float16).to(dev)
            cbr = (torch.randn(256, 8, generator=g) * 0.02).to(torch.float16).to(dev)
            pm = zipf(g, 65536, cnt).to(torch.int32).to(torch.int16).view(torch.uint8)
            pr = zipf(g, 256, cnt).to(torch.uint8)
            rsc = (torch.rand(nn_, generator=g) + 0.5).to(torch.float16).to(dev)
            rbi = (torch.randn(nn_, generator=g) * 0.01).to(torch.float16).to(dev)
            rot = rot_for(pm.numel() + pr.numel(), cap=128)
            pms = [pm.to(dev).clone() for _ in range(rot)]
            prs = [pr.to(dev).clone() for _ in range(rot)]
            w32 = kernels.rvq_dequant(pms[0], 16, prs[0], 8, cbm, cbr, rsc, rbi, nn_, kk, torch.float16).float()
            alg4 = lambda m: cnt * 3 + (65536 + 256) * 16 + nn_ * 4 + m * kk * 2 + m * nn_ * 2
            for m, band in ((1, "a:fused-gemv"), (32, "a:fused-gemv"), (128, "b:tile-gemm"), (384, "b:tile-gemm"),
                            (384, "c:decode+gemm")):
                xm = xpair(m, kk, 40 + m, torch.float16)
                if band == "a:fused-gemv":
                    f = lambda i: kernels.rvq_linear(xm[i % 2], pms[i], 16, prs[i], 8, cbm, cbr, rsc, rbi, nn_)
                elif band == "b:tile-gemm":
                    f = lambda i: kernels.rvq_linear(xm[i % 2], pms[i], 16, prs[i], 8, cbm, cbr, rsc, rbi, nn_, tile=True)
                else:
                    f = lambda i: torch.nn.functional.linear(
                        xm[i % 2], kernels.rvq_dequant(pms[i], 16, prs[i], 8, cbm, cbr, rsc, rbi, nn_, kk, torch.float16))
                run(f"cfg4 rvq {nn_}x{kk} f16", band, m, f, rot, alg4(m), 2.0 * m * nn_ * kk, ref=lambda: xm[0].float() @ w32.T)
            del pms, prs, w32
            torch.cuda.empty_cache()
        # config 5: int4 group-affine, fp16, both shapes
        from neuropress_amd.t2n.packing import BitPacking4

        for nn_, kk in ((14336, 4096), (4096, 4096)):
            g = gen(1005)
            blob = BitPacking4.compress(torch.randint(0, 16, (nn_, kk), generator=g, dtype=torch.int64).to(torch.uint8))
            sc = (torch.rand(nn_ * kk // 32, generator=g) * 0.019 + 0.001).to(torch.float16).to(dev)
            rot = rot_for(blob.numel(), cap=128)
            blobs = [blob.to(dev)]
            blobs += [blobs[0].clone() for _ in range(rot - 1)]
            w32 = kernels.q_dequant(blobs[0], sc, 4, 32, None, torch.float16).float()
            for m in (1, 16, 32, 256) + ((384, 512) if nn_ == 14336 else ()):
                xm = xpair(m, kk, 90 + m, torch.float16)
                algq = nn_ * kk // 2 + nn_ * kk // 32 * 2 + m * kk * 2 + m * nn_ * 2
                run(f"cfg5 int4 {nn_}x{kk} f16", "a:gemv" if m <= 32 else "b:tile-gemm", m,
                    lambda i: kernels.q_linear(xm[i % 2], blobs[i], sc, 4, 32), rot, algq, 2.0 * m * nn_ * kk,
                    ref=lambda: xm[0].float() @ w32.T)
                if m >= 256:
                    run(f"cfg5 int4 {nn_}x{kk} f16", "c:decode+gemm", m, lambda i: torch.nn.functional.linear(
                        xm[i % 2], kernels.q_dequant(blobs[i], sc, 4, 32, None, torch.float16)), rot, algq,
                        2.0 * m * nn_ * kk, ref=lambda: xm[0].float() @ w32.T)
            if nn_ == 14336:
                q5 = {"blob": blob, "scale": sc.cpu(), "x": xpair(1, kk, 91, torch.float16)[0].cpu(), "n": nn_, "k": kk,
                      "y": kernels.q_linear(xpair(1, kk, 91, torch.float16)[0], blobs[0], sc, 4, 32).cpu()}
            del blobs, w32
            torch.cuda.empty_cache()
        # neighbours of the linear on a decode step: RMSNorm and the embedding lookups (Llama-3-8B sizes)
        hdim, vocab = 4096, 128256
        wn = (torch.rand(hdim, generator=g) + 0.5).to(torch.bfloat16).to(dev)
        for m in (1, 4096):
            xn = [torch.randn(m, hdim, generator=gen(95 + i)).to(torch.bfloat16).to(dev) for i in range(8 if m > 1 else 2)]
            run("rms_norm H=4096 bf16", "aux", m, lambda i: kernels.rms_norm(xn[i % len(xn)], wn, 1e-6), len(xn),
                2 * m * hdim * 2 + hdim * 2, 0.0, steps=20)
        cbe = (torch.randn(65536, 8, generator=g) * 0.02).to(torch.float16).to(dev)
        tab = torch.randint(0, 65536, (vocab, hdim // 8), generator=g, dtype=torch.int32).to(torch.int16).to(dev)
        qblob = torch.randint(0, 256, (vocab, hdim // 2), generator=g, dtype=torch.int32).to(torch.uint8).to(dev)
        qsc = (torch.rand(vocab * hdim // 32, generator=g) * 0.019 + 0.001).to(torch.float16).to(dev)
        for m in (1, 4096):
            ids = [torch.randint(0, vocab, (m,), generator=gen(97 + i)).to(dev) for i in range(4)]
            run("vq_embedding 128256x4096 -> bf16", "aux", m,
                lambda i: kernels.vq_embedding(ids[i % 4], tab, cbe, 64.0, None, torch.bfloat16), 4,
                m * (8 + hdim // 8 * 2 + hdim // 8 * 16 + hdim * 2), 0.0, steps=20)
            run("int4 embedding 128256x4096 -> bf16", "aux", m,
                lambda i: kernels.q_embedding(ids[i % 4], qblob, qsc, 4, 32, None, None, 64.0, torch.bfloat16), 4,
                m * (8 + hdim // 2 + hdim // 32 * 2 + hdim * 2), 0.0, steps=20)
        del tab, qblob, qsc
        torch.cuda.empty_cache()
    result["sweep"] = sweep

    # ---------------- CPU baseline: the reference's CPU path, same workloads ------
    if not args.no_cpu:
        from oracle import torch_path  # test infrastructure, used here only as the timed CPU baseline

        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        torch.set_num_threads(cores)
        cpu_model = host_cpu_description()

        def median_ms(fn):
            """(median seconds, last result): 1-2 warm-up calls, then 5 timed (fewer when one call is slow)."""
            t0 = time.perf_counter()
            out = fn()
            first = time.perf_counter() - t0
            if first < 0.5:
                fn()
            reps = []
            for _ in range(5 if first < 0.5 else 3 if first < 1.5 else 1):
                t0 = time.perf_counter()
                out = fn()
                reps.append(time.perf_counter() - t0)
            return sorted(reps)[len(reps) // 2], out, len(reps)

        def leg(name, variant, decode, x_cpu, alg_bytes, y_gpu):
            t_dec, w_cpu, it = median_ms(decode)
            t_mm, y_cpu, _ = median_ms(lambda: torch.nn.functional.linear(x_cpu, w_cpu))
            entry = {"case": name, "variant": variant, "cores": cores, "kind": "port",
                     "decode_ms": round(t_dec * 1e3, 2), "matmul_ms": round(t_mm * 1e3, 2),
                     "ms_per_call": round((t_dec + t_mm) * 1e3, 2), "timed_iterations": it,
                     "value": round(alg_bytes / (t_dec + t_mm) / 1e9, 3), "unit": "GB/s"}
            if y_gpu is not None:
                entry["gpu_matches_cpu_within_1e-2"], entry["max_abs_diff"] = check_against_cpu(y_gpu, y_cpu)
            return entry

        x_cpu = xs[0].cpu()
        cpu_rows = [
            leg("cfg3 14336x4096 bf16 M=1", "vectorised unpack (16-bit view) + gather + cast, F.linear",
                lambda: torch_path.vq_decode_cpu(c3["packed"], c3["cb"], 16, n, k, torch.bfloat16, True),
                x_cpu, alg, ys[0]),
            leg("cfg3 14336x4096 bf16 M=1", "per-bit loop unpack (reference-faithful) + gather + cast, F.linear",
                lambda: torch_path.vq_decode_cpu(c3["packed"], c3["cb"], 16, n, k, torch.bfloat16, False),
                x_cpu, alg, ys[0]),
            leg("cfg3 14336x4096 bf16 M=384", "vectorised unpack (16-bit view) + gather + cast, F.linear",
                lambda: torch_path.vq_decode_cpu(c3["packed"], c3["cb"], 16, n, k, torch.bfloat16, True),
                x384_cpu, vq_alg_bytes(c3, 384), None),
        ]
        if not args.no_sweep:
            cpu_rows.append(
                leg("cfg5 int4 14336x4096 f16 M=1", "nibble shifts + (q - 8) * scale + cast, F.linear",
                    lambda: torch_path.q_decode_cpu(q5["blob"], q5["scale"], 4, 32, torch.float16),
                    q5["x"], q5["n"] * q5["k"] // 2 + q5["n"] * q5["k"] // 32 * 2 + q5["k"] * 2 + q5["n"] * 2, q5["y"]))
        head = cpu_rows[0]
        result["cpu_baselines"] = cpu_rows
        result["cpu_baseline"] = {
            "value": head["value"], "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "the full config-3 up/gate layer at M=1: median of 5 calls each of the decode (16-bit view + "
                      "codebook gather + cast to bf16) and of torch F.linear in bf16",
            "ms_per_call": head["ms_per_call"], "decode_ms": head["decode_ms"], "matmul_ms": head["matmul_ms"],
            "cpu": cpu_model,
            "gpu_matches_cpu_within_1e-2": head["gpu_matches_cpu_within_1e-2"], "max_abs_diff": head["max_abs_diff"],
        }
    result["roofline"] = roofline
    result["roofline_m384"] = roofline_m384
    result["checks"] = checks
    print(json.dumps(result))


if __name__ == "__main__":
    main()
