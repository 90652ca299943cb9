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
T, NUM_DELTAS, BITS, GROUP = 32, 8, 2, -1    # the default workload (configuration 2)


# HBM bytes per launch (average over the 4 launches of a step) of the default workload, from
# rocprofv3 FETCH_SIZE and WRITE_SIZE runs of this script, each scaled by what the same counter
# reads for the --calib-copy-mib copy kernel.  The figure belongs to the kernel sources it was
# measured on: it is reported only while their fingerprint (kernel_fingerprint) still equals the
# one recorded here with the profile, and withheld (null) once the kernel has changed.
MEASURED_TRAFFIC = {
    "bytes_per_launch": 212437042,
    "profile": "profiles/dz_mdl32_kernel__llama7b_decode_t32_d8_2bit__hbm_traffic.txt",
    "kernel_sha256": "d96f2d8b27debcd2f6491b9da047a29acc594bb7a6ff0ba52ca2b2f965cb572a",
}
KERNEL_SOURCES = ("deltazip_amd/csrc/dz_mdl32.hip", "deltazip_amd/csrc/dz_device.h", "deltazip_amd/csrc/dz_layout.h")


def kernel_fingerprint():
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


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
    xd, idd, wbd = torch.from_numpy(x).to(dev), torch.from_numpy(ids).to(dev), torch.from_numpy(wb).to(dev)
    ref = o.forward_ref(x, wb, dts, ids)
    y = ops.apply_delta(xd, q, s, m, idd, wbd)
    yt = ops.apply_delta(xd, q, s, m, idd, wbd, base_tiled=ops.tile_base(wbd))   # the form the timed loop reads
    err = max(o.rel_err(y.cpu().numpy(), ref), o.rel_err(yt.cpu().numpy(), ref))
    same = bool(torch.equal(y, yt))
    return {"dequant_bit_exact": bool(exact), "max_rel_err": float(err), "tolerance": 1e-2,
            "tiled_base_equals_row_major": same, "ok": bool(exact and same and err <= 1e-2)}


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.lower().startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline():
    """The reference's CPU path (unpack -> dequant -> W_base + delta in fp32 -> matmul per id) on
    this host.  Per distinct layer shape: 3 untimed calls, then the median of 5; a step is
    4 + 2 + 1 such calls.  Reported: all threads with the dequantisation on every call (what the
    naive reference does; `value`), all threads with the deltas dequantised beforehand (matmul
    only, a lower bound), and one thread (smallest shape only, scaled by weight elements)."""
    from oracle import cpu_path
    g = torch.Generator().manual_seed(7)
    ids = torch.sort(torch.randint(0, NUM_DELTAS, (T,), generator=g)).values
    nthreads = torch.get_num_threads()

    def timed(fn, warm, reps):
        for _ in range(warm):
            fn()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return float(np.median(ts))

    per_shape, per_shape_mm, total, total_mm, one_thread = {}, {}, 0.0, 0.0, None
    step_elems = sum(K * N for _, K, N in SHAPES)
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
        dt = timed(lambda: cpu_path.forward_cpu(x, wb, deltas, ids, BITS), 3, 5)
        pre = [cpu_path.dequant_torch(*d, BITS) for d in deltas]
        dm = timed(lambda: cpu_path.forward_cpu(x, wb, deltas, ids, BITS, predequantised=pre), 3, 5)
        per_shape[f"{K}x{N}"], per_shape_mm[f"{K}x{N}"] = dt, dm
        total += count * dt
        total_mm += count * dm
        if one_thread is None:
            torch.set_num_threads(1)
            try:
                d1 = timed(lambda: cpu_path.forward_cpu(x, wb, deltas, ids, BITS), 1, 3)
            finally:
                torch.set_num_threads(nthreads)
            one_thread = {"threads": 1, "seconds_4096x4096": d1,
                          "tokens_per_s_extrapolated": T / (d1 * step_elems / (K * N)),
                          "sample": "4096x4096 only, 1 untimed call + median of 3; step time scaled by weight "
                                    "elements (x%.2f)" % (step_elems / (K * N))}
        del deltas, pre
    return {"value": T / total, "unit": "tokens/s", "cores": nthreads, "kind": "port",
            "sample": "each distinct projection shape (4096x4096, 4096x11008, 11008x4096): 3 untimed calls, "
                      "median of 5; dequant + fp32 add + matmul per delta on every call, as the naive "
                      "reference does; step time = 4*t1 + 2*t2 + t3",
            "seconds_per_step": total, "seconds_per_shape": per_shape,
            "matmul_only": {"value": T / total_mm, "unit": "tokens/s", "seconds_per_step": total_mm,
                            "seconds_per_shape": per_shape_mm,
                            "what": "deltas dequantised beforehand; fp32 add + matmul per delta (lower bound)"},
            "one_thread": one_thread, "cpu_model": _cpu_model(), "os_cpu_count": os.cpu_count()}


SHAPES_13B = [("q_proj", 5120, 5120), ("k_proj", 5120, 5120), ("v_proj", 5120, 5120), ("o_proj", 5120, 5120),
              ("gate_proj", 5120, 13824), ("up_proj", 5120, 13824), ("down_proj", 13824, 5120)]
MFMA_F16_PEAK_TFLOPS = 2500.0

# BASELINE.json's configurations.  The default (and the one the metric is quoted on) is 2; the
# others are parity-test cases that can also be timed here with --config.
CONFIGS = {
    1: dict(name="4096->4096, 1 token, one 4-bit delta (per-channel scales)", shapes=[("linear", 4096, 4096)],
            T=1, S=1, bits=4, gs=-1, ids="zeros", bound="hbm"),
    2: dict(name="Llama-2-7B decode projections (q,k,v,o 4096->4096; gate,up 4096->11008; down 11008->4096), "
                 "one step = these 7 multi-delta linears (q/k/v in one launch, gate/up in one launch, as the "
                 "reference's fused layers run them; --separate-launches: 7 launches); 32 tokens, 8 deltas (2-bit, 2:4 sparse, "
                 "per-channel fp16 scales), ids uniform over the deltas",
            shapes=SHAPES, T=32, S=8, bits=2, gs=-1, ids="uniform", bound="hbm"),
    3: dict(name="Llama-2-7B projections, 64 tokens, 32 deltas (4-bit, 2:4, group size 128), Zipf(1.5) ids",
            shapes=SHAPES, T=64, S=32, bits=4, gs=128, ids="zipf", bound="hbm"),
    4: dict(name="Llama-2-13B prefill projections, 16 requests x 512 tokens, each bound to its own delta "
                 "(2-bit, 2:4, per-channel)", shapes=SHAPES_13B, T=8192, S=16, bits=2, gs=-1, ids="blocks",
            bound="mfma"),
    5: dict(name="one full decode step of a random-init 32-layer Llama-2-7B (hidden 4096, 32 heads, FFN 11008, "
                 "fp16): every projection (fused q/k/v, o, fused gate/up, down) is a multi-delta layer created by "
                 "the delta manager; RMSNorm, rotary and attention over a 1024-token KV context are plain "
                 "PyTorch-ROCm ops; embedding and output projection on the base tables; 128 decode tokens, "
                 "64 resident deltas (2-bit, 2:4 sparse, per-channel scales), ids uniform over the deltas",
            shapes=SHAPES, T=128, S=64, bits=2, gs=-1, ids="uniform", bound="hbm"),
}


def make_ids(kind, t, s, dev, gen, sort):
    if kind == "zeros":
        return torch.zeros(t, dtype=torch.int64, device=dev)
    if kind == "blocks":
        return torch.repeat_interleave(torch.arange(s, device=dev), t // s)
    if kind == "zipf":
        p = torch.arange(1, s + 1, device=dev, dtype=torch.float32) ** -1.5
        ids = torch.multinomial(p / p.sum(), t, replacement=True, generator=gen)
    else:
        ids = torch.randint(0, s, (t,), device=dev, generator=gen)
    return torch.sort(ids).values if sort else ids   # the serving scheduler delivers batches sorted by delta id


def timed_steps(step, steps, warmup, min_warm_seconds=0.25):
    """At least `warmup` untimed steps and at least `min_warm_seconds` of them (so that the clocks
    have ramped whatever --warmup says), then exactly `steps` timed ones between two events on the
    current stream and two synchronisations -- nothing else is put on the stream inside the timed
    region (an event per step costs about 8 us of a 170 us step: the marker waits for the kernel
    before it and holds back the one after it).  The per-step times (sorted, ms) come from a second
    pass of `steps` steps with an event in front of each, after the timed region.
    Returns (wall seconds, event seconds, sorted per-step ms, warm steps run)."""
    done, t_w = 0, time.perf_counter()
    while done < warmup or time.perf_counter() - t_w < min_warm_seconds:
        for _ in range(max(1, min(50, warmup - done))):
            step(done)
            done += 1
        torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        step(i)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    for i in range(steps):
        evs[i].record()
        step(i)
    evs[steps].record()
    torch.cuda.synchronize()
    return (wall, e0.elapsed_time(e1) * 1e-3,
            sorted(evs[i].elapsed_time(evs[i + 1]) for i in range(steps)), done)


def run_full_step(args, parity):
    """Configuration 5: the whole decode step (deltazip_amd/llama_step.py) with every projection a
    multi-delta layer; reports the step, the share of the projections in it and their HBM fraction."""
    from deltazip_amd import DeltaConfig, DeltaMapping, create_delta_manager
    from deltazip_amd.llama_step import LlamaForDecodeStep, LlamaStepConfig
    from deltazip_amd.synthetic import gaussian_native_stack, random_native_stack
    cfg = CONFIGS[5]
    T, S, bits, gs, ctx = cfg["T"], cfg["S"], cfg["bits"], cfg["gs"], 1024
    steps, warmup = args.steps or 10, args.warmup or 2
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(1234)
    mcfg = LlamaStepConfig(num_hidden_layers=args.layers or 32)
    model = LlamaForDecodeStep(mcfg, device=dev, generator=gen)
    mgr = create_delta_manager(model, max_num_seqs=T, max_num_batched_tokens=T, vocab_size=mcfg.vocab_size,
                               delta_config=DeltaConfig(max_deltas=S, max_bitwidth=bits, group_size=gs,
                                                        tile_base_weights=not args.row_major_base,
                                                        keep_row_major_base=args.row_major_base))
    # synthetic deltas (N(0, 1e-3), compressed on the GPU) written straight into the layers' slot stacks;
    # the manager is told that delta d + 1 lives in slot d
    make_stack = random_native_stack if args.random_bits else gaussian_native_stack
    for name, layer in mgr.modules.items():
        N, K = layer.base_shape
        layer.qweight_stacked, layer.meta_stacked, layer.scales_stacked = make_stack(K, N, bits, gs, S, dev, gen)
        layer.bitwidth = [bits] * S
    mgr.delta_index_to_id = list(range(1, S + 1))
    ids = torch.sort(torch.randint(1, S + 1, (T,), device=dev, generator=gen)).values.tolist()
    mgr.set_delta_mapping(DeltaMapping(tuple(ids), tuple(ids)))
    d_present = len(set(ids))
    tokens = torch.randint(0, mcfg.vocab_size, (T,), device=dev, generator=gen)
    kv = model.make_kv_cache(T, ctx, dev)
    torch.cuda.synchronize()

    wall, gpu_s, step_ms, warm_run = timed_steps(lambda i: model.decode_step(tokens, kv, ctx), steps, warmup)
    ms_per_step = wall / steps * 1e3

    # the projections alone: the same 4 x layers calls on inputs of the right shape
    projs = [m for _, m in model.projections()]
    xs = {K: torch.randn((T, K), device=dev, dtype=torch.float16, generator=gen)
          for K in {m.base_shape[1] for m in projs}}

    def linears(i):
        for m in projs:
            m(xs[m.base_shape[1]])
    lwall, lgpu, _, _ = timed_steps(linears, steps, warmup)
    lin_ms = lgpu / steps * 1e3
    lin_bytes = sum(algorithmic_bytes(m.base_shape[1], m.base_shape[0], T, bits, d_present) for m in projs)
    nbytes = lambda t: t.numel() * t.element_size()
    footprint = {
        "base_projection_weights_bytes": sum(nbytes(m.base_layer.weight) + (nbytes(m.base_tiled) if m.base_tiled is not None
                                                                              else 0) for m in projs),
        "base_projection_copies": "tiles only (the row-major weight is freed once the tiles are made: "
                                  "DeltaConfig.keep_row_major_base=False)" if not args.row_major_base else "row-major only",
        "delta_slots_bytes": sum(nbytes(m.qweight_stacked) + nbytes(m.meta_stacked) + nbytes(m.scales_stacked) for m in projs),
        "kv_cache_bytes": sum(nbytes(k_) + nbytes(v_) for k_, v_ in kv),
        "allocated_bytes": torch.cuda.memory_allocated(), "reserved_bytes": torch.cuda.memory_reserved(),
        "hbm_bytes": torch.cuda.get_device_properties(0).total_memory}
    achieved = lin_bytes / (lin_ms * 1e-3) / 1e9
    out = {
        "metric": "multi-delta linear tokens/s + achieved HBM TB/s (% peak), Llama-7B shapes",
        "value": T / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step, "ms_per_step_median": round(step_ms[steps // 2], 4), "warmup_steps_run": warm_run,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic (random-init model; " + ("delta slots filled with uniformly random bits)" if args.random_bits
                                                     else "deltas ~ N(0, 1e-3) compressed on the GPU)"),
        "config": {"workload": cfg["name"] + ", batch sorted by delta id", "baseline_config": 5, "tokens": T,
                   "deltas": S, "deltas_present": d_present, "bits": bits, "group_size": gs, "kv_context": ctx,
                   "layers": mcfg.num_hidden_layers, "launches_per_step": len(projs),
                   "base_weight_layout": "row-major [N, K]" if args.row_major_base
                                         else "tiles (dz_tile_base, converted once when the layer is created)"},
        "linear_layers": {"ms_per_step": round(lin_ms, 4), "share_of_step": round(lin_ms / (gpu_s / steps * 1e3), 4),
                          "calls": len(projs), "us_per_call": round(lin_ms * 1e3 / len(projs), 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "dz_mdl32_kernel (the projections of the step, timed on their own)",
                     "algorithmic_bytes_per_launch": lin_bytes // len(projs),
                     "avg_launch_us": round(lin_ms * 1e3 / len(projs), 2)},
        "hbm_footprint": footprint,
        "parity": parity,
    }
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=0, help="timed steps (default 200; 10 for --config 4)")
    ap.add_argument("--warmup", type=int, default=0, help="untimed steps (default 20; 2 for --config 4)")
    ap.add_argument("--config", type=int, default=2, choices=sorted(CONFIGS), help="BASELINE.json configuration")
    ap.add_argument("--layers", type=int, default=0, help="distinct decoder layers kept in HBM and visited in turn "
                                                       "(--config 5: decoder layers of the model, default 32)")
    ap.add_argument("--unsorted", action="store_true", help="do not sort the batch by delta id")
    ap.add_argument("--row-major-base", action="store_true",
                    help="read the base weight as the plain [N, K] tensor instead of the tiled copy a layer makes of it")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--random-bits", action="store_true",
                    help="fill the delta slots with uniformly random code and position bits instead of compressing "
                         "N(0, sigma) deltas (the configured workload)")
    ap.add_argument("--no-probe", action="store_true", help="skip the yardstick launches (read-only probe; library GEMM)")
    ap.add_argument("--no-qualifiers", action="store_true",
                    help="default workload: skip the extra timed loops on the unsorted batch and the row-major base "
                         "weight (counter runs: every dispatch of the kernel then belongs to the headline workload)")
    ap.add_argument("--ksplit", type=int, default=0)
    ap.add_argument("--separate-launches", action="store_true",
                    help="one launch per projection (default: q/k/v and gate/up, which share their input in a "
                         "decoder layer and which the reference holds as fused layers, go in one launch each)")
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
    from deltazip_amd.synthetic import gaussian_native_stack, random_native_stack
    cfg = CONFIGS[args.config]
    shapes, T, S, bits, gs = cfg["shapes"], cfg["T"], cfg["S"], cfg["bits"], cfg["gs"]
    steps = args.steps or (10 if args.config == 4 else 200)
    warmup = args.warmup or (2 if args.config == 4 else 20)
    nlayers = args.layers or {1: 16, 2: 4, 3: 2, 4: 1, 5: 32}[args.config]
    lib = _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    gen = torch.Generator(device=dev).manual_seed(1234)

    parity = parity_check(dev)
    if args.config == 5:
        return run_full_step(args, parity)

    # ---- resident inputs
    # up to 128 tokens the layer reads its base weight from the tiled copy it makes at creation
    # (dz_tile_base); --row-major-base measures the fused kernel on the plain [N, K] weight instead
    fused = T <= 128
    if not fused and not args.separate_launches and [sh[0] for sh in shapes] == [sh[0] for sh in SHAPES]:
        # prefill-sized calls: q/k/v and gate/up are one layer each, with one weight and one stacked delta
        # over the fused output dimension -- how the merged layers hold and run them
        # (serving/vllm/delta/layers_marlin.py:281-487)
        (_, K0, Nq), (_, _, Nk), (_, _, Nv), o, (_, _, Ng), (_, _, Nu), down = shapes
        shapes = [("q+k+v", K0, Nq + Nk + Nv), o, ("gate+up", K0, Ng + Nu), down]
    tiled_base = not args.row_major_base
    default_workload = (args.config == 2 and not args.unsorted and args.ksplit == 0 and not args.separate_launches
                        and not args.row_major_base)
    ids = make_ids(cfg["ids"], T, S, dev, gen, not args.unsorted)
    d_present = int(torch.unique(ids).numel())
    sigma = 2e-3 if args.config == 1 else 1e-3
    layers = []
    for li in range(nlayers):
        calls = []
        for si, (name, K, N) in enumerate(shapes):
            if args.random_bits:
                q, m, s = random_native_stack(K, N, bits, gs, S, dev, gen)
            else:
                # the deltas the configuration describes: N(0, sigma), scales from the un-pruned values,
                # 2:4 by magnitude, quantised -- compressed on the GPU (seeded per configuration, layer, shape)
                dgen = torch.Generator(device=dev).manual_seed(1000 * args.config + 100 * li + si)
                q, m, s = gaussian_native_stack(K, N, bits, gs, S, dev, dgen, sigma)
            wb = (torch.randn((N, K), device=dev, generator=gen) * 0.02).half()
            wbt = ops.tile_base(wb) if (fused or tiled_base) else None     # as a layer does once when it is created
            if fused and not default_workload:
                # only one form is read in this run (the default workload also times the other one)
                if tiled_base:
                    wb = None
                else:
                    wbt = None
            x = torch.randn((T, K), device=dev, generator=gen).half()
            y = torch.empty((T, N), dtype=torch.float16, device=dev)
            calls.append((name, K, N, x, wb, q, m, s, y, wbt))
        layers.append(calls)
    stream = torch.cuda.current_stream().cuda_stream
    ops.set_ksplit(args.ksplit)

    # launches of a step: q/k/v in one, o, gate/up in one, down (the reference runs q/k/v and gate/up as
    # fused layers: serving/vllm/delta/layers_marlin.py:281-487); --separate-launches: one per projection
    names = [sh[0] for sh in shapes]
    groups = [[j] for j in range(len(shapes))]
    if fused and not args.separate_launches and names == [sh[0] for sh in SHAPES]:
        groups = [[0, 1, 2], [3], [4, 5], [6]]

    vp = C.c_void_p
    keep = []                                   # the pointer arrays must outlive the calls
    if fused:
        ws_bytes = max(lib.dz_workspace_bytes(T, shapes[g[0]][1], sum(shapes[j][2] for j in g)) for g in groups)
        ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)
        # 33..128 tokens: the order in which the kernel takes the tokens depends on the ids only; it is
        # computed once per step (inside the timed region) and every launch of the step reuses it, as the
        # reference converts its mapping once per batch
        order = torch.empty(T, dtype=torch.int32, device=dev) if T > 32 else None

        def marshal(tiled, ids_t):
            """Pre-marshalled C-ABI calls (device pointers and sizes only): per layer the launches of a
            step, and every projection as a launch of its own (per-shape timing)."""
            fb = lib.dz_multi_delta_linear_batch_tiled if tiled else lib.dz_multi_delta_linear_batch
            prepared, single = [], []
            for calls in layers:
                def batch_args(g):
                    n = len(g)
                    arr = lambda k: (vp * n)(*[calls[j][k].data_ptr() for j in g])
                    ax, aw, aq, am, asc, ay = arr(3), arr(9 if tiled else 4), arr(5), arr(6), arr(7), arr(8)
                    an = (C.c_int * n)(*[calls[j][2] for j in g])
                    keep.append((ax, aw, aq, am, asc, ay, an))
                    return (n, ax, aw, aq, am, asc, vp(ids_t.data_ptr()), ay, an, an, T, calls[g[0]][1], S, bits,
                            gs, 0, vp(order.data_ptr()) if order is not None else None,
                            vp(ws.data_ptr()), C.c_size_t(ws_bytes), vp(stream))
                prepared.append([(fb, batch_args(g)) for g in groups])
                single.append([(fb, batch_args([j])) for j in range(len(calls))])
            return prepared, single

        prepared, single = marshal(tiled_base, ids)

        def launch(i, gi, prep=None):
            fn, a = (prep or prepared)[i % len(layers)][gi]
            rc = fn(*a)
            if rc:
                raise RuntimeError(f"multi-delta linear launch failed: {lib.dz_strerror(rc).decode()}")

        def call(i, idx):
            launch(i, idx, single)
    else:
        # prefill-sized: the batch is ordered by delta and cut into row blocks once per step (inside the
        # timed region; as the reference converts its mapping once per batch), then one launch of the
        # packed-delta GEMM per layer
        order = None
        blocks = [None]

        def call(i, idx):
            name, K, N, x, wb, q, m, s, y, wbt = layers[i % len(layers)][idx]
            ops.multi_delta_linear(x, None if tiled_base else wb, q, s, m, ids, bits=bits, out=y, order=blocks[0],
                                   base_tiled=wbt if tiled_base else None)

        def launch(i, gi, prep=None):
            call(i, groups[gi][0])

    def make_step(prep=None, ids_t=None):
        ids_t = ids if ids_t is None else ids_t

        def step(i):
            if not fused:
                blocks[0] = ops.row_blocks(ids_t, S)
            if fused and order is not None:
                rc = lib.dz_token_order(C.c_void_p(ids_t.data_ptr()), T, S, C.c_void_p(order.data_ptr()), C.c_void_p(stream))
                if rc:
                    raise RuntimeError(f"dz_token_order failed: {lib.dz_strerror(rc).decode()}")
            for gi in range(len(groups)):
                launch(i, gi, prep)
        return step
    step = make_step()

    if args.calib_copy_mib > 0:
        src = torch.ones(args.calib_copy_mib << 19, dtype=torch.float16, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)         # one elementwise kernel: reads src once, writes dst once
        torch.cuda.synchronize()
        del src, dst

    wall, gpu_s, step_ms, warm_steps_run = timed_steps(step, steps, warmup)
    median_step_ms = step_ms[steps // 2]

    def abytes(K, N):
        return algorithmic_bytes(K, N, T, bits, d_present, 1 if gs == -1 else K // gs)
    launches = steps * len(groups)
    step_bytes = sum(abytes(K, N) for _, K, N in shapes)
    step_flops = sum(2.0 * T * K * N for _, K, N in shapes)
    avg_launch_s = gpu_s / launches              # includes the gaps between consecutive launches
    ms_per_step = wall / steps * 1e3

    # per-shape time (event pairs around single calls, outside the timed region)
    per_call_us = {}
    for (K, N) in dict.fromkeys((K, N) for _, K, N in shapes):
        idx = [j for j, sh in enumerate(shapes) if (sh[1], sh[2]) == (K, N)][0]
        ts = []
        for i in range(12 if fused else 4):
            s0, s1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s0.record(); call(i, idx); s1.record(); torch.cuda.synchronize()
            ts.append(s0.elapsed_time(s1) * 1e3)
        us = float(np.median(ts[2:]))
        b = abytes(K, N)
        ent = {"us": round(us, 2), "GBps": round(b / us / 1e3, 1), "frac": round(b / us / 1e3 / HBM_PEAK_GBPS, 3)}
        if cfg["bound"] == "mfma":
            ent = {"us": round(us, 2), "TFLOPs": round(2.0 * T * K * N / us / 1e6, 1),
                   "frac": round(2.0 * T * K * N / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 3)}
        per_call_us[f"{K}x{N}"] = ent

    def time_loop(fn, iters, warm=12):
        """us per call of fn(i) over `iters` back-to-back calls on the current stream (HIP events)."""
        for i in range(warm):
            fn(i)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for i in range(iters):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / iters

    if cfg["bound"] == "hbm":
        achieved = (step_bytes / len(groups)) / avg_launch_s / 1e9
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBPS, 4),
                    "traffic": (MEASURED_TRAFFIC["bytes_per_launch"]
                                if default_workload and MEASURED_TRAFFIC["kernel_sha256"] == kernel_fingerprint() else None),
                    "traffic_profile": MEASURED_TRAFFIC["profile"],
                    "kernel": "dz_mdl32_kernel" if all(len(g) == 1 for g in groups) else "dz_mdl32_kernel + dz_mdl32_batch_kernel (same body)",
                    "algorithmic_bytes_per_launch": step_bytes // len(groups),
                    "avg_launch_us": round(avg_launch_s * 1e6, 2)}
        if default_workload and not args.no_qualifiers:
            # the two qualifiers of the headline, measured in the same run on the same weights: the batch
            # as drawn (not sorted by delta id), and the base weight read as the plain [N, K] tensor
            reps = max(50, min(steps, 200))
            ids_u = make_ids(cfg["ids"], T, S, dev, torch.Generator(device=dev).manual_seed(1234), False)
            prep_u, _ = marshal(True, ids_u)
            us_u = time_loop(make_step(prep_u, ids_u), reps)
            prep_r, _ = marshal(False, ids)
            us_r = time_loop(make_step(prep_r), reps)
            roofline["unsorted_frac"] = round(step_bytes / us_u / 1e3 / HBM_PEAK_GBPS, 4)
            roofline["row_major_frac"] = round(step_bytes / us_r / 1e3 / HBM_PEAK_GBPS, 4)
            roofline["unsorted_ms_per_step"] = round(us_u * 1e-3, 5)
            roofline["row_major_ms_per_step"] = round(us_r * 1e-3, 5)
        if fused and tiled_base and T <= 32 and not args.no_probe and all(len(g) <= 4 for g in groups):
            # Yardstick: for every launch of the step, a read-only launch with the same grid that makes
            # the same 16-byte streaming requests for the tiled base weight and the packed words of the
            # deltas present -- no ids, no arithmetic, no exchange of partial sums, no output -- and
            # the fused launch timed the same way (back to back, rotating over the resident layers).
            sink = torch.zeros(64, dtype=torch.int32, device=dev)
            dpr = min(d_present, 8)
            pp = {}
            pargs = []
            for gi, g in enumerate(groups):
                pa = []
                for calls in layers:
                    n = len(g)
                    arr = lambda k: (vp * n)(*[calls[j][k].data_ptr() for j in g])
                    ax, aw, aq, am = arr(3), arr(9), arr(5), arr(6)
                    an = (C.c_int * n)(*[calls[j][2] for j in g])
                    keep.append((ax, aw, aq, am, an))
                    pa.append((n, ax, aw, aq, am, an, T, shapes[g[0]][1], bits, dpr))
                pargs.append(pa)

            def probe(i, gi, with_x):
                rc = lib.dz_probe_read(*pargs[gi][i % len(layers)], with_x, vp(sink.data_ptr()), vp(stream))
                if rc:
                    raise RuntimeError(f"dz_probe_read failed: {lib.dz_strerror(rc).decode()}")

            def probe_step(i, with_x):
                for gi in range(len(groups)):
                    probe(i, gi, with_x)
            # the whole step as read-only launches, in the step's own order over the same resident layers
            # (same footprint per pass as the timed loop: nothing is found in the last-level cache)
            reps = max(50, min(steps, 200))
            probe_step_us = {wx: time_loop(lambda i: probe_step(i, wx), reps) for wx in (0, 1)}
            fused_step_us = time_loop(step, reps)
            for gi, g in enumerate(groups):
                K = shapes[g[0]][1]
                wbytes = sum(2 * K * shapes[j][2] + dpr * (K * shapes[j][2] * bits // 16 + K * shapes[j][2] // 8) for j in g)
                abytes_g = sum(abytes(shapes[j][1], shapes[j][2]) for j in g)
                us0 = time_loop(lambda i: probe(i, gi, 0), 60)
                us1 = time_loop(lambda i: probe(i, gi, 1), 60)
                usf = time_loop(lambda i: launch(i, gi), 60)
                pp["+".join(names[j] for j in g)] = {
                    "weight_bytes": wbytes, "algorithmic_bytes": abytes_g,
                    "read_only_us": round(us0, 2), "read_only_frac_of_peak": round(wbytes / us0 / 1e3 / HBM_PEAK_GBPS, 4),
                    "read_only_with_activation_requests_us": round(us1, 2),
                    "fused_us": round(usf, 2), "fused_frac_of_peak": round(abytes_g / usf / 1e3 / HBM_PEAK_GBPS, 4),
                    "fused_over_read_only": round(us0 / usf, 4)}
            roofline["practical_peak"] = {
                "what": "read-only launches with the fused kernel's grids and 16-byte streaming requests (dz_probe_read): "
                        "no ids, no arithmetic, no exchange, no output; each launch timed back to back like the fused one",
                "per_launch_note": "each launch repeated back to back over the resident layers: a smaller footprint per "
                                   "pass than the step's, so part of it may be found in the last-level cache; the step "
                                   "figures below are the yardstick",
                "per_launch": pp,
                "step_read_only_us": round(probe_step_us[0], 2),
                "step_read_only_with_activation_requests_us": round(probe_step_us[1], 2),
                "step_fused_us": round(fused_step_us, 2),
                "frac": round(step_bytes / probe_step_us[0] / 1e3 / HBM_PEAK_GBPS, 4),
                "fused_over_read_only": round(probe_step_us[0] / fused_step_us, 4)}
    else:
        # base contraction only (2*T*K*N per call); the per-delta dequantisation and the delta half of
        # the pair-GEMM are extra work inside the same time
        achieved = (step_flops / len(groups)) / avg_launch_s / 1e12
        roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(achieved / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None,
                    "kernel": "dz_gemm24_kernel", "algorithmic_flops_per_call": step_flops / len(groups),
                    "avg_call_us": round(avg_launch_s * 1e6, 2)}
        if not args.no_probe:
            # Yardstick: the library's dense fp16 GEMM (torch.mm -> hipBLASLt / rocBLAS) on the same base
            # weights and activations, in the step's order over the same resident layers -- the base half
            # of the work alone, no delta.  The fused kernel issues 1.5 matrix instructions per base one
            # (a 16x16x64 sparse product for every two dense 16x16x32), so its rate in issued matrix
            # instructions is 1.5 x its rate in base flops.
            def lib_step(i):
                for name, K, N, x, wb, q, m, s, y, _ in layers[i % len(layers)]:
                    torch.mm(x, wb.t(), out=y)
            us_lib = time_loop(lib_step, max(4, min(steps, 20)), warm=3)
            us_own = time_loop(step, max(4, min(steps, 20)), warm=3)
            lib_tf = step_flops / us_lib / 1e6
            own_tf = step_flops / us_own / 1e6
            roofline["practical_peak"] = {
                "what": "torch.mm (the ROCm GEMM library) on the same base weights and activations: dense fp16 "
                        "base product only, no delta; both timed back to back the same way",
                "library_step_us": round(us_lib, 1), "library_tflops": round(lib_tf, 1),
                "library_frac_of_peak": round(lib_tf / MFMA_F16_PEAK_TFLOPS, 4),
                "fused_step_us": round(us_own, 1), "fused_base_tflops": round(own_tf, 1),
                "fused_matrix_instruction_tflops_equivalent": round(1.5 * own_tf, 1) if bits == 2 else None,
                "fused_over_library": round(us_lib / us_own, 4)}

    out = {
        "metric": "multi-delta linear tokens/s + achieved HBM TB/s (% peak), Llama-7B shapes",
        "value": T / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step,
        "ms_per_step_median": round(median_step_ms, 5), "ms_per_step_min": round(step_ms[0], 5),
        "warmup_steps_run": warm_steps_run,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic" + (" (delta slots filled with uniformly random bits)" if args.random_bits else
                               " (deltas ~ N(0, %g) compressed on the GPU: scales from the un-pruned values, 2:4 by "
                               "magnitude, %d-bit codes; base ~ N(0, 0.02), x ~ N(0, 1))" % (sigma, bits)),
        "config": {"workload": cfg["name"] + ("" if args.unsorted or cfg["ids"] in ("zeros", "blocks")
                                              else ", batch sorted by delta id"),
                   "baseline_config": args.config, "tokens": T, "deltas": S, "deltas_present": d_present,
                   "bits": bits, "group_size": gs, "layers_resident": nlayers, "launches_per_step": len(groups),
                   "launches": ["+".join(names[j] for j in g) for g in groups],
                   "base_weight_layout": "tiles (dz_tile_base, converted once like the deltas)" if tiled_base
                                         else "row-major [N, K]"},
        "us_per_layer_call": round(gpu_s / (steps * len(shapes)) * 1e6, 2),
        "per_shape": per_call_us,
        "roofline": roofline,
        "parity": parity,
    }
    if not args.no_cpu_baseline and args.config == 2:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
