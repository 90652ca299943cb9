#!/usr/bin/env python3
"""Benchmark of the multi-delta linear layer on one MI355X.

Workload (BASELINE.json configs[1]): the seven projections of one Llama-2-7B decoder layer
(q, k, v, o: 4096->4096; gate, up: 4096->11008; down: 11008->4096), 32 decode tokens whose
delta ids are uniform over 8 resident deltas, every delta 2-bit, 2:4 sparse, per-channel fp16
scales, base weights fp16.  One step = those seven layer calls on one batch.  The weights of
several decoder layers are kept in HBM and visited in turn, so that no call finds its weights in
the last-level cache.  All inputs are in HBM before the timed region starts.

Prints one JSON line: tokens/s through the seven multi-delta linears of a decoder layer, the
achieved fraction of the 8 TB/s HBM roofline (algorithmic bytes, see `algorithmic_bytes`), and the
reference's CPU path timed on this host's cores on a bounded sample.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
SHAPES = [("q_proj", 4096, 4096), ("k_proj", 4096, 4096), ("v_proj", 4096, 4096), ("o_proj", 4096, 4096),
          ("gate_proj", 4096, 11008), ("up_proj", 4096, 11008), ("down_proj", 11008, 4096)]   # (name, K, N)
T, NUM_DELTAS, BITS, GROUP = 32, 8, 2, -1


# HBM bytes per launch (average over the 7 launches of a step) of the default workload, from
# rocprofv3 FETCH_SIZE and WRITE_SIZE runs of this script, each scaled by what the same counter
# reads for the --calib-copy-mib copy kernel; the figures are in profiles/*__hbm_traffic.txt.
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = 123460880


def algorithmic_bytes(K, N, T, bits, d_present, G=1):
    """Bytes one layer call has to move: base fp16 once; per distinct delta present its codes
    (kept half, `bits` each), a 2-bit position per kept value and the fp16 scales; activations in,
    outputs out, int64 ids."""
    return 2 * K * N + d_present * (K * N * bits // 16 + K * N // 8 + 2 * G * N) + 2 * T * K + 2 * T * N + 8 * T


def parity_check(dev):
    """Small same-run parity gate against the CPU oracle: dequant bit-exact, output rel err."""
    from oracle import dz_oracle as o
    from deltazip_amd import ops
    n, k, nd = 512, 4096, 8
    qs, ms, ss, dts = [], [], [], []
    for d in range(nd):
        dl = o.make_delta(n, k, 1e-3, BITS, GROUP, 2000 + d)
        q, m, s = ops.repack_gptq_to_native(*(torch.from_numpy(dl[key]) for key in ("qweight", "qzeros", "scales", "g_idx")), BITS)
        qs.append(q); ms.append(m); ss.append(s)
        dts.append(o.dequant_gptq(dl["qweight"], dl["qzeros"], dl["scales"], dl["g_idx"], BITS))
    q, m, s = (torch.stack(v).to(dev) for v in (qs, ms, ss))
    exact = all(np.array_equal(ops.dequant(q[d], m[d], s[d], k, n, BITS).cpu().numpy().view(np.uint16),
                               np.ascontiguousarray(dts[d].T).view(np.uint16)) for d in range(nd))
    wb, x = o.make_base(n, k, 2000), o.make_x(T, k, 2500)
    ids = np.sort(o.make_ids("uniform", T, nd, 2900))
    y = ops.apply_delta(torch.from_numpy(x).to(dev), q, s, m, torch.from_numpy(ids).to(dev), torch.from_numpy(wb).to(dev))
    err = o.rel_err(y.cpu().numpy(), o.forward_ref(x, wb, dts, ids))
    return {"dequant_bit_exact": bool(exact), "max_rel_err": float(err), "tolerance": 1e-2,
            "ok": bool(exact and err <= 1e-2)}


def cpu_baseline():
    """The reference's CPU path (unpack -> dequant -> W_base + delta in fp32 -> matmul per id) on
    this host, one call of each distinct layer shape; a step is 4 + 2 + 1 such calls."""
    from oracle import cpu_path
    g = torch.Generator().manual_seed(7)
    ids = torch.sort(torch.randint(0, NUM_DELTAS, (T,), generator=g)).values
    per_shape, total = {}, 0.0
    for (K, N), count in (((4096, 4096), 4), ((4096, 11008), 2), ((11008, 4096), 1)):
        pf = 32 // BITS
        deltas = []
        for _ in range(NUM_DELTAS):
            qw = torch.randint(-2 ** 31, 2 ** 31 - 1, (K // pf, N), dtype=torch.int32, generator=g)
            qz = torch.full((1, N // pf), 0x55555555, dtype=torch.int32)
            sc = (torch.rand((1, N), generator=g) * 1e-3 + 2e-4).half()
            deltas.append((qw, qz, sc, torch.zeros(K, dtype=torch.int32)))
        wb = (torch.randn((N, K), generator=g) * 0.02).half()
        x = torch.randn((T, K), generator=g).half()
        reps = []
        for _ in range(3):                       # first call warms the allocator and BLAS threads
            t0 = time.perf_counter()
            cpu_path.forward_cpu(x, wb, deltas, ids, BITS)
            reps.append(time.perf_counter() - t0)
        dt = float(np.median(reps[1:]))
        per_shape[f"{K}x{N}"] = dt
        total += count * dt
    return {"value": T / total, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "each distinct projection shape (4096x4096, 4096x11008, 11008x4096) called 3 times, "
                      "median of the last 2; dequant + fp32 add + matmul per delta on every call, as the "
                      "naive reference does; step time = 4*t1 + 2*t2 + t3",
            "seconds_per_step": total, "seconds_per_shape": per_shape, "os_cpu_count": os.cpu_count()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--layers", type=int, default=4, help="distinct decoder layers kept in HBM and visited in turn")
    ap.add_argument("--unsorted", action="store_true", help="do not sort the batch by delta id")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--ksplit", type=int, default=0)
    ap.add_argument("--calib-copy-mib", type=int, default=0,
                    help="before the timed region, run a plain elementwise copy kernel over this many MiB "
                         "(reads and writes that much): the yardstick for scaling FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU fallback for the measured path)", file=sys.stderr)
        sys.exit(2)
    from deltazip_amd import _lib, ops
    from deltazip_amd.synthetic import random_native_stack
    lib = _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(1234)

    parity = parity_check(dev)

    # ---- resident inputs
    ids = torch.randint(0, NUM_DELTAS, (T,), device=dev, generator=gen)
    if not args.unsorted:
        ids = torch.sort(ids).values            # the serving scheduler delivers batches sorted by delta id
    d_present = int(torch.unique(ids).numel())
    layers = []
    for _ in range(args.layers):
        calls = []
        for name, K, N in SHAPES:
            q, m, s = random_native_stack(K, N, BITS, GROUP, NUM_DELTAS, dev, gen)
            wb = (torch.randn((N, K), device=dev, generator=gen) * 0.02).half()
            x = torch.randn((T, K), device=dev, generator=gen).half()
            y = torch.empty((T, N), dtype=torch.float16, device=dev)
            calls.append((name, K, N, x, wb, q, m, s, y))
        layers.append(calls)
    ws_bytes = max(lib.dz_workspace_bytes(T, K, N) for _, K, N in SHAPES)
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    ops.set_ksplit(args.ksplit)

    # pre-marshalled C-ABI calls (device pointers and sizes only)
    f = lib.dz_multi_delta_linear
    vp = C.c_void_p
    prepared = []
    for calls in layers:
        pc = []
        for name, K, N, x, wb, q, m, s, y in calls:
            pc.append((vp(x.data_ptr()), vp(wb.data_ptr()), vp(q.data_ptr()), vp(m.data_ptr()), vp(s.data_ptr()),
                       vp(ids.data_ptr()), vp(y.data_ptr()), T, K, N, NUM_DELTAS, BITS, GROUP, 0, N,
                       vp(ws.data_ptr()), C.c_size_t(ws_bytes), vp(stream)))
        prepared.append(pc)

    def step(i):
        for a in prepared[i % len(prepared)]:
            rc = f(*a)
            if rc:
                raise RuntimeError(f"dz_multi_delta_linear failed: {lib.dz_strerror(rc).decode()}")

    if args.calib_copy_mib > 0:
        src = torch.ones(args.calib_copy_mib << 19, dtype=torch.float16, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)         # one elementwise kernel: reads src once, writes dst once
        torch.cuda.synchronize()
        del src, dst

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()                                  # on the stream the kernels are launched on
    for i in range(args.steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    gpu_s = e0.elapsed_time(e1) * 1e-3

    default_workload = not args.unsorted and args.ksplit == 0
    launches = args.steps * len(SHAPES)
    step_bytes = sum(algorithmic_bytes(K, N, T, BITS, d_present) for _, K, N in SHAPES)
    avg_launch_s = gpu_s / launches              # includes the gaps between consecutive launches
    achieved = (step_bytes / len(SHAPES)) / avg_launch_s / 1e9
    ms_per_step = wall / args.steps * 1e3

    # per-shape kernel time (event pairs around single launches, outside the timed region)
    per_call_us = {}
    for name, K, N in (("4096x4096", 4096, 4096), ("4096x11008", 4096, 11008), ("11008x4096", 11008, 4096)):
        idx = [j for j, sh in enumerate(SHAPES) if (sh[1], sh[2]) == (K, N)][0]
        ts = []
        for i in range(12):
            a = prepared[i % len(prepared)][idx]
            s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s0.record(); f(*a); s1.record(); torch.cuda.synchronize()
            ts.append(s0.elapsed_time(s1) * 1e3)
        us = float(np.median(ts[2:]))
        b = algorithmic_bytes(K, N, T, BITS, d_present)
        per_call_us[name] = {"us": round(us, 2), "GBps": round(b / us / 1e3, 1), "frac": round(b / us / 1e3 / HBM_PEAK_GBPS, 3)}

    out = {
        "metric": "multi-delta linear tokens/s + achieved HBM TB/s (% peak), Llama-7B shapes",
        "value": T / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "Llama-2-7B decode projections (q,k,v,o 4096->4096; gate,up 4096->11008; "
                               "down 11008->4096), one step = these 7 multi-delta linear calls; 32 tokens, "
                               "8 deltas (2-bit, 2:4 sparse, per-channel fp16 scales), ids uniform over the deltas"
                               + ("" if args.unsorted else ", batch sorted by delta id"),
                   "tokens": T, "deltas": NUM_DELTAS, "deltas_present": d_present, "bits": BITS,
                   "layers_resident": args.layers, "launches_per_step": len(SHAPES)},
        "us_per_layer_call": round(avg_launch_s * 1e6, 2),
        "per_shape": per_call_us,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH if default_workload else None,
                     "kernel": "dz_mdl32_kernel<2,2,false>",
                     "algorithmic_bytes_per_launch": step_bytes // len(SHAPES),
                     "avg_launch_us": round(avg_launch_s * 1e6, 2)},
        "parity": parity,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
