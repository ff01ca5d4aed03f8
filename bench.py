#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

Headline workload (BASELINE.json configs[1]): int4 weight-only decode GEMV, M=1, K=4096,
N=11008, group 128, fp16 activations / scales / zeros, weights in the reference's packed device
layout.  One "step" = one call of the GEMV on weights that are NOT cache resident: the calls walk
round-robin through enough distinct copies of the packed weight (> 512 MiB) that every call
streams its 24 MB from HBM.  The K timed steps are recorded into one HIP graph and replayed once,
so launch gaps do not dilute the kernel time; the region is bracketed by HIP events on the launch
stream and by device synchronisation.

Prints ONE JSON line (see the keys at the bottom).  `value` is GB/s of algorithmic bytes
(packed nibbles + scales/zeros + activations + outputs = 23,983,616 B per call).  `extras` carries
the other kernels of the path (int8 GEMM TOPS at 2048x4096x4096 with the fused dequant epilogue,
activation quantizer, ternary matmul, batched int4).  `cpu_baseline` times the CPU oracle's port of
the reference's CPU int4 kernel on the host cores, on the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "int4 GEMV GB/s (% HBM peak) at M=1; int8 GEMM TOPS (% MFMA peak) at M=2048"
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0        # MI355X dense int8 MFMA
M, K, N, GROUP = 1, 4096, 11008, 128
GEMV_BYTES = N * K // 2 + (K // GROUP) * N * 4 + 2 * M * K + 2 * M * N   # 23,983,616
GEMV_PROFILE = os.path.join(ROOT, "profiles", "int4_decode_gemv_M1_K4096_N11008.md")
INT8_PROFILE = os.path.join(ROOT, "profiles", "int8_gemm_stagger_M2048_K4096_N4096.md")


def measured_traffic_bytes(profile=None):
    """HBM bytes per launch of the GEMV kernel (or of the kernel of another profile summary) as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (each scaled by
    what the same counter reads for a 256 MiB device copy, --calibrate-copy).  The figure lives in the committed profile
    summary, on a line `traffic_bytes_per_launch: <bytes> (commit <hash>)`; None when that file or line is missing."""
    import re

    try:
        m = re.search(r"^traffic_bytes_per_launch:\s*(\d+)", open(profile or GEMV_PROFILE).read(), flags=re.M)
    except OSError:
        return None
    return int(m.group(1)) if m else None


def asym_quant_int4(w, group):
    """Asymmetric uint4 group quantizer of the benchmark configuration: s = (max-min)/15,
    q = clamp(round((w-min)/s), 0, 15), zero = min + 8 s, so (q-8)*s + zero = min + q*s."""
    import numpy as np

    n, k = w.shape
    wg = w.reshape(n, k // group, group)
    lo, hi = wg.min(-1), wg.max(-1)
    s = np.maximum((hi - lo) / 15.0, 1e-8).astype(np.float32)
    q = np.clip(np.rint((wg - lo[..., None]) / s[..., None]), 0, 15).astype(np.int32).reshape(n, k)
    z = (lo + 8 * s).astype(np.float32)
    return q, np.ascontiguousarray(np.stack([s.T, z.T], axis=-1))  # [K/g, N, 2]


def time_region(fn, stream_sync, reps):
    """Run fn() `reps` times between two HIP events on the current stream; returns ms per call."""
    import torch

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    stream_sync()
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    stream_sync()
    return start.elapsed_time(stop) / reps


def steady(fn, stream_sync, reps=1, warm_ms=30.0, batches=7):
    """fn() repeated for at least `warm_ms` of wall time (after host-side set-up the chip needs about 20 ms of
    work to reach its sustained clocks), then the median over `batches` timed regions of `reps` calls; ms per call."""
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < warm_ms:
        for _ in range(reps):
            fn()
        stream_sync()
    return sorted(time_region(fn, stream_sync, reps) for _ in range(batches))[batches // 2]


def graph_of(fn):
    """Record fn() (which only enqueues kernels on the current stream) into a HIP graph."""
    import torch

    g = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(g):  # switches the current stream to a capturing side stream
        fn()
    return g


def load_probe():
    """The pure-read measurement probe: a library of its own (tensorplay_amd/csrc/probe.hip), not part of the kernel
    library's interface."""
    import ctypes

    from tensorplay_amd import build

    if not os.path.exists(build.PROBE_LIB_PATH):
        raise RuntimeError(f"{build.PROBE_LIB_PATH} is missing: build it with `python -m tensorplay_amd.build`")
    lib = ctypes.CDLL(build.PROBE_LIB_PATH)
    lib.tpq_probe_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.tpq_probe_read.restype = ctypes.c_int
    return lib


def host_description():
    """What the CPU baseline ran on: logical CPUs the OS reports, CPUs this process may use, physical cores, model name
    and the ISA tier that decides the reference's CPU int4 layout (64-column blocks on AVX-512, 32 on AVX2 / plain)."""
    info = {"os_cpu_count": os.cpu_count()}
    try:
        info["usable_cpus"] = len(os.sched_getaffinity(0))
    except AttributeError:
        info["usable_cpus"] = os.cpu_count()
    model, flags, cores = None, set(), set()
    try:
        phys = core = None
        for line in open("/proc/cpuinfo"):
            key, _, val = line.partition(":")
            key, val = key.strip(), val.strip()
            if key == "model name" and model is None:
                model = val
            elif key == "flags" and not flags:
                flags = set(val.split())
            elif key == "physical id":
                phys = val
            elif key == "core id":
                core = val
            elif not key and phys is not None and core is not None:
                cores.add((phys, core))
                phys = core = None
    except OSError:
        pass
    info["cpu_model"] = model
    info["physical_cores"] = len(cores) or None
    info["isa_tier"] = "avx512" if "avx512f" in flags else "avx2" if "avx2" in flags else "default"
    return info


def cpu_baseline(x16, codes, sz16, want, budget_s=8.0):
    """The CPU oracle's port of the reference's CPU int4 kernel (AVX-512 layout, 4-row x 64-column tasks spread over
    threads), timed on the host on the full M=1 workload at two thread counts: every CPU this process may use (the
    box gives a one-GPU job a share of the host, so that is capped at 16) and 4, the default of the reference's own
    benchmark (benchmark/bench_quantized_native.py:181).  The timed library is the oracle's source compiled with
    -march=native on this host; if that build fails the portable AVX2 build is timed and the record says so."""
    import tempfile

    import numpy as np

    import oracle

    host = host_description()
    native, build = None, "gcc -O3 -march=native"
    try:
        native = oracle.build_native(tempfile.mkdtemp(prefix="tpq_oracle_"))
    except Exception as exc:  # no compiler on the host: the library that travelled with the repository
        build = f"portable build (-mavx2 -mfma); native build failed: {str(exc)[:80]}"
    packed = oracle.int4_pack_cpu(codes, 64, True)
    blocks = N // 64

    def timed(threads, budget):
        out = np.zeros((M, N), np.uint16)
        per = (blocks + threads - 1) // threads
        spans = [(b, min(b + per, blocks)) for b in range(0, blocks, per)]
        pool = ThreadPoolExecutor(max_workers=threads)

        def call():
            list(pool.map(lambda sp: oracle.int4_mm_cpu_blocked(x16, "f16", packed, sz16, GROUP, sp, out, library=native), spans))

        call()
        err = float(np.abs(oracle.to_f32(out, "f16") - want).max() / np.abs(want).max())
        t0 = time.perf_counter()
        calls = 0
        while True:
            call()
            calls += 1
            dt = time.perf_counter() - t0
            if dt > budget or calls >= 2000:
                break
        pool.shutdown()
        return dt / calls, calls, err

    all_threads = max(1, min(16, host["usable_cpus"] or 1))
    per_call, calls, err = timed(all_threads, budget_s)
    per_call4, calls4, _ = timed(min(4, all_threads), budget_s / 2)
    # the library twin the reference benchmarks its CPU op against (test_native_operator_families.py:579-599):
    # PyTorch's own CPU int4 kernel on the same codes, default thread count, a few seconds
    twin = None
    try:
        import torch

        if hasattr(torch, "_weight_int4pack_mm_for_cpu"):
            szt = torch.from_numpy(sz16.view(np.float16).astype(np.float32)).half()
            xt = torch.from_numpy(x16.view(np.float16).copy())
            pk = torch._convert_weight_to_int4pack_for_cpu(torch.from_numpy(codes.astype(np.int32)), 1)
            torch._weight_int4pack_mm_for_cpu(xt, pk, GROUP, szt)
            t1 = time.perf_counter()
            n_twin = 0
            while time.perf_counter() - t1 < 3.0:
                torch._weight_int4pack_mm_for_cpu(xt, pk, GROUP, szt)
                n_twin += 1
            twin = {"GBs": round(GEMV_BYTES / ((time.perf_counter() - t1) / n_twin) / 1e9, 3), "threads": torch.get_num_threads()}
    except Exception as exc:  # the twin is a side figure: never fail the benchmark over it
        twin = {"error": str(exc)[:120]}
    return {
        "torch_cpu_twin": twin,
        "value": round(GEMV_BYTES / per_call / 1e9, 3),
        "unit": "GB/s",
        "cores": all_threads,
        "kind": "port",
        "sample": f"{calls} calls of the full M=1 K=4096 N=11008 GEMV ({per_call * 1e6:.0f} us/call), "
                  f"oracle port of the reference CPU int4 kernel; max rel diff vs GPU {err:.2e}",
        "four_threads": {"value": round(GEMV_BYTES / per_call4 / 1e9, 3), "unit": "GB/s", "cores": min(4, all_threads),
                         "sample": f"{calls4} calls ({per_call4 * 1e6:.0f} us/call)"},
        "host": host,
        "build": build,
        "layout": "64-column blocks, half-split nibbles (the reference's AVX-512 tier)",
    }


def decoder_layer_share(dev, rng_seed=5):
    """BASELINE configs[4]: one Llama-style decoder layer (d=4096, 32 heads x 128, MLP 11008, SwiGLU,
    RMSNorm eps 1e-5, interleaved RoPE, no biases, as in the reference's benchmark/bench_llama_e2e.py:37-92),
    all seven projections int4 group-128 weight-only, decode step at batch 8 against a 2048-token fp16
    KV cache.  Attention, norms, RoPE and the elementwise glue are PyTorch-ROCm fp16 ops; the seven
    linears are this library's.  Three copies of the layer's weights rotate so that they are read from
    HBM, as they would be in a 32-layer model.  Returns layer us, linears-only us and the share."""
    import torch
    import torch.nn.functional as F

    from tensorplay_amd.ao.quantization import WeightOnlyInt4Linear

    d, H, D, inter, B, T = 4096, 32, 128, 11008, 8, 2048
    gen = torch.Generator(device=dev).manual_seed(rng_seed)
    shapes = {"q": (d, d), "k": (d, d), "v": (d, d), "o": (d, d), "gate": (inter, d), "up": (inter, d), "down": (d, inter)}
    copies = 3
    layers = []
    for _ in range(copies):
        mods = {}
        for name, (n, k) in shapes.items():
            lin = torch.nn.Linear(k, n, bias=False, device=dev, dtype=torch.float16)
            with torch.no_grad():
                lin.weight.copy_((torch.randn(n, k, device=dev, generator=gen) * 0.02).half())
            mods[name] = WeightOnlyInt4Linear.from_float(lin, 128)
            del lin
        layers.append(mods)
    torch.cuda.empty_cache()
    n1 = torch.ones(d, device=dev, dtype=torch.float16)
    n2 = torch.ones(d, device=dev, dtype=torch.float16)
    kc = (torch.randn(B, H, T + 1, D, device=dev, generator=gen) * 0.5).half()
    vc = (torch.randn(B, H, T + 1, D, device=dev, generator=gen) * 0.5).half()
    x0 = torch.randn(B, 1, d, device=dev, generator=gen).half()
    inv = 1.0 / (10000.0 ** (torch.arange(D // 2, device=dev, dtype=torch.float32) * 2.0 / D))
    ang = float(T) * inv
    cos, sin = ang.cos().half().view(1, 1, 1, D // 2), ang.sin().half().view(1, 1, 1, D // 2)

    def rope(t):
        e, o = t[..., 0::2], t[..., 1::2]
        return torch.stack((e * cos - o * sin, e * sin + o * cos), dim=-1).reshape_as(t)

    def layer(L, x):
        r = x
        xn = F.rms_norm(x, (d,), n1, 1e-5)
        q = L["q"](xn).view(B, 1, H, D).transpose(1, 2)
        k = L["k"](xn).view(B, 1, H, D).transpose(1, 2)
        v = L["v"](xn).view(B, 1, H, D).transpose(1, 2)
        q, k = rope(q), rope(k)
        kc[:, :, T:T + 1] = k
        vc[:, :, T:T + 1] = v
        a = F.scaled_dot_product_attention(q, kc, vc)
        x = r + L["o"](a.transpose(1, 2).reshape(B, 1, H * D))
        r = x
        xn = F.rms_norm(x, (d,), n2, 1e-5)
        return r + L["down"](F.silu(L["gate"](xn)) * L["up"](xn))

    from tensorplay_amd import ops as tops

    def layer_fused(L, x):
        """The same layer with q, k and v in one launch and the two fusions around the MLP matmuls: residual add
        in the epilogue of the o and down projections, gate and up in one launch with the SwiGLU epilogue."""
        xf = x.view(B, d)
        xn = F.rms_norm(xf, (d,), n1, 1e-5)
        q, k, v = tops.int4pack_mm_multi(xn, [L[n].weight for n in "qkv"], 128, [L[n].scales_and_zeros for n in "qkv"])
        q, k, v = (t.view(B, 1, H, D).transpose(1, 2) for t in (q, k, v))
        q, k = rope(q), rope(k)
        kc[:, :, T:T + 1] = k
        vc[:, :, T:T + 1] = v
        a = F.scaled_dot_product_attention(q, kc, vc).transpose(1, 2).reshape(B, H * D)
        x1 = tops.int4pack_mm_add(a, L["o"].weight, 128, L["o"].scales_and_zeros, xf)
        xn = F.rms_norm(x1, (d,), n2, 1e-5)
        h = tops.int4pack_mm_swiglu(xn, L["gate"].weight, L["up"].weight, 128, L["gate"].scales_and_zeros, L["up"].scales_and_zeros)
        return tops.int4pack_mm_add(h, L["down"].weight, 128, L["down"].scales_and_zeros, x1).view(B, 1, d)

    def layer_fused_norm(L, x):
        """layer_fused with the two RMS norms inside the launches that consume them (q, k, v; gate and up)."""
        xf = x.view(B, d)
        q, k, v = tops.int4pack_mm_multi(xf, [L[n].weight for n in "qkv"], 128, [L[n].scales_and_zeros for n in "qkv"],
                                         norm_weight=n1, eps=1e-5)
        q, k, v = (t.view(B, 1, H, D).transpose(1, 2) for t in (q, k, v))
        q, k = rope(q), rope(k)
        kc[:, :, T:T + 1] = k
        vc[:, :, T:T + 1] = v
        a = F.scaled_dot_product_attention(q, kc, vc).transpose(1, 2).reshape(B, H * D)
        x1 = tops.int4pack_mm_add(a, L["o"].weight, 128, L["o"].scales_and_zeros, xf)
        h = tops.int4pack_mm_swiglu(x1, L["gate"].weight, L["up"].weight, 128, L["gate"].scales_and_zeros, L["up"].scales_and_zeros,
                                    norm_weight=n2, eps=1e-5)
        return tops.int4pack_mm_add(h, L["down"].weight, 128, L["down"].scales_and_zeros, x1).view(B, 1, d)

    xin = {n: torch.randn(B, 1, k, device=dev, generator=gen).half() for n, (_, k) in shapes.items()}
    res_d = torch.randn(B, d, device=dev, generator=gen).half()

    def linears_fused(L):
        tops.int4pack_mm_multi(xin["q"].view(B, d), [L[n].weight for n in "qkv"], 128, [L[n].scales_and_zeros for n in "qkv"])
        tops.int4pack_mm_add(xin["o"].view(B, d), L["o"].weight, 128, L["o"].scales_and_zeros, res_d)
        tops.int4pack_mm_swiglu(xin["gate"].view(B, d), L["gate"].weight, L["up"].weight, 128, L["gate"].scales_and_zeros,
                                L["up"].scales_and_zeros)
        tops.int4pack_mm_add(xin["down"].view(B, inter), L["down"].weight, 128, L["down"].scales_and_zeros, res_d)

    def linears_fused_norm(L):
        tops.int4pack_mm_multi(xin["q"].view(B, d), [L[n].weight for n in "qkv"], 128, [L[n].scales_and_zeros for n in "qkv"],
                               norm_weight=n1, eps=1e-5)
        tops.int4pack_mm_add(xin["o"].view(B, d), L["o"].weight, 128, L["o"].scales_and_zeros, res_d)
        tops.int4pack_mm_swiglu(xin["gate"].view(B, d), L["gate"].weight, L["up"].weight, 128, L["gate"].scales_and_zeros,
                                L["up"].scales_and_zeros, norm_weight=n2, eps=1e-5)
        tops.int4pack_mm_add(xin["down"].view(B, inter), L["down"].weight, 128, L["down"].scales_and_zeros, res_d)

    def linears(L):
        for name in shapes:
            L[name](xin[name])

    reps = 12
    out = layer(layers[0], x0)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    out_f = layer_fused(layers[0], x0)
    torch.cuda.synchronize()
    fused_diff = float((out_f.float() - out.float()).abs().max() / out.float().abs().max())
    assert fused_diff < 2e-2, fused_diff
    out_n = layer_fused_norm(layers[0], x0)
    torch.cuda.synchronize()
    norm_diff = float((out_n.float() - out.float()).abs().max() / out.float().abs().max())
    assert norm_diff < 2e-2, norm_diff
    g_layer = graph_of(lambda: [layer(layers[i % copies], x0) for i in range(reps)])
    g_lin = graph_of(lambda: [linears(layers[i % copies]) for i in range(reps)])
    g_layer_f = graph_of(lambda: [layer_fused(layers[i % copies], x0) for i in range(reps)])
    g_lin_f = graph_of(lambda: [linears_fused(layers[i % copies]) for i in range(reps)])
    g_layer_n = graph_of(lambda: [layer_fused_norm(layers[i % copies], x0) for i in range(reps)])
    g_lin_n = graph_of(lambda: [linears_fused_norm(layers[i % copies]) for i in range(reps)])
    res = {"layer_fused_vs_unfused_max_rel_diff": fused_diff, "layer_fused_norm_vs_unfused_max_rel_diff": norm_diff}
    for key, g in (("layer_decode_b8_kv2048_us", g_layer), ("layer_int4_linears_us", g_lin),
                   ("layer_decode_fused_mlp_us", g_layer_f), ("layer_int4_linears_fused_us", g_lin_f),
                   ("layer_decode_fused_mlp_norm_us", g_layer_n), ("layer_int4_linears_fused_norm_us", g_lin_n)):
        g.replay(); torch.cuda.synchronize()
        res[key] = steady(g.replay, torch.cuda.synchronize) / reps * 1e3
    res["layer_int4_linear_share"] = res["layer_int4_linears_us"] / res["layer_decode_b8_kv2048_us"]
    lin_bytes = sum(n * k // 2 + (k // 128) * n * 4 + 2 * B * k + 2 * B * n for n, k in shapes.values())
    res["layer_int4_linears_GBs"] = lin_bytes / (res["layer_int4_linears_us"] * 1e-6) / 1e9
    res["layer_int4_linears_fused_GBs"] = lin_bytes / (res["layer_int4_linears_fused_us"] * 1e-6) / 1e9
    return res


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the host CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="time the headline GEMV only")
    ap.add_argument("--gemv-only", action="store_true", help="extras of the int4 GEMV only (no int8 / quantizer / ternary)")
    ap.add_argument("--no-layer", action="store_true", help="skip the decoder-layer share measurement (config 5)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a plain 256 MiB device copy a few times: the known-size kernel that "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings are scaled by")
    ap.add_argument("--profile-rows", type=int, default=0, metavar="M",
                    help="also launch the int4 product at M activation rows (same weights, rotating) 200 times, eagerly: "
                         "the dispatches that the rocprofv3 summaries of the batched-decode kernels are collected on")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from tensorplay_amd import _lib, ops

    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    sync = torch.cuda.synchronize

    def cur():  # the stream to launch on: the capturing stream while a graph is being recorded
        return torch.cuda.current_stream().cuda_stream

    # ---- synthetic workload (seeded) -------------------------------------------------------
    rng = np.random.default_rng(20260101)
    w = rng.normal(0, 0.02, (N, K)).astype(np.float32)
    codes, sz = asym_quant_int4(w, GROUP)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    x_d = torch.from_numpy(x).to(dev).half()
    sz_d = torch.from_numpy(sz).to(dev).half().contiguous()
    packed0 = ops._convert_weight_to_int4pack(torch.from_numpy(codes).to(dev), 2)
    copies = 64  # 64 x (22.5 + 1.4) MB = 1.53 GB: far beyond L2 + the 256 MB last-level cache
    packs = [packed0] + [packed0.clone() for _ in range(copies - 1)]
    szs = [sz_d] + [sz_d.clone() for _ in range(copies - 1)]
    y_d = torch.empty((M, N), dtype=torch.float16, device=dev)

    ws = torch.zeros(lib.tpq_int4_mm_workspace_bytes(N), dtype=torch.uint8, device=dev)

    def gemv(i):
        rc = lib.tpq_int4_mm_ws(x_d.data_ptr(), _lib.F16, M, K, packs[i % copies].data_ptr(), 2, N, GROUP,
                                szs[i % copies].data_ptr(), y_d.data_ptr(), ws.data_ptr(), ws.numel(), cur())
        if rc:
            raise RuntimeError(_lib.last_error())

    # correctness of what is being timed (fp64 evaluation of the same quantized weights)
    gemv(0)
    sync()
    sz16 = sz_d.cpu().view(torch.int16).numpy().view(np.uint16)
    x16 = x_d.cpu().view(torch.int16).numpy().view(np.uint16)
    sz32 = sz_d.float().cpu().numpy().astype(np.float64)
    wq = (codes - 8) * np.repeat(sz32[:, :, 0].T, GROUP, axis=1) + np.repeat(sz32[:, :, 1].T, GROUP, axis=1)
    want = x_d.float().cpu().numpy().astype(np.float64) @ wq.T
    got = y_d.float().cpu().numpy()
    gpu_err = float(np.abs(got - want).max() / np.abs(want).max())
    if not gpu_err < 1e-3:
        raise RuntimeError(f"int4 GEMV output is off by {gpu_err:.3e} (limit 1e-3)")

    # ---- headline: W warmup steps, then exactly K timed steps ------------------------------------
    steps, warmup = max(1, args.steps), max(0, args.warmup)
    for i in range(warmup):
        gemv(i)
    sync()
    g = graph_of(lambda: [gemv(i) for i in range(steps)])
    g.replay()  # untimed: first replay uploads the graph
    sync()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    sync()
    t0 = time.perf_counter()
    start.record()
    g.replay()
    stop.record()
    sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = start.elapsed_time(stop) / steps
    gbs = GEMV_BYTES / (ms_per_step * 1e-3) / 1e9

    extras = {"gemv_max_rel_err_vs_fp64": gpu_err, "graph_wall_ms_per_step": wall_ms / steps}
    roofline_int8 = None
    if not args.no_extras:  # the same graph seven more times: median step time
        reps = sorted(time_region(g.replay, sync, 1) / steps for _ in range(7))
        extras["int4_gemv_us_median_of_7_replays"] = reps[3] * 1e3
        # Is the start-up of the K-step figure the host submitting the graph while the GPU idles behind the start event?
        # The same K-step graph with the GPU still busy when the host gets there (a replay of it directly in front, no
        # synchronization between).  It reads the same (6.58 against 6.59 us at 20 steps): the start-up of about 9 us
        # belongs to every graph launch on the GPU side, whatever the host does.
        def busy_start():
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            sync()
            g.replay()
            a.record()
            g.replay()
            b.record()
            sync()
            return a.elapsed_time(b) / steps
        extras["int4_gemv_us_K_steps_gpu_busy_at_start"] = sorted(busy_start() for _ in range(7))[3] * 1e3
        # The K-step graph above carries its own start-up (about half a microsecond per step at 20 steps).  The same
        # kernel timed the way every other figure here is: a graph of 640 launches, warmed for >= 30 ms, median of 7.
        gs = graph_of(lambda: [gemv(i) for i in range(10 * copies)])
        gs.replay(); sync()
        steady_us = steady(gs.replay, sync) / (10 * copies) * 1e3
        extras["int4_gemv_steady_us"] = steady_us
        extras["int4_gemv_steady_GBs"] = GEMV_BYTES / (steady_us * 1e-6) / 1e9
        extras["int4_gemv_steady_frac_of_hbm_peak"] = GEMV_BYTES / (steady_us * 1e-6) / 1e9 / HBM_PEAK_GBS
        extras["int4_gemv_steady_launches_per_graph"] = 10 * copies
        del gs
    if not args.no_extras:
        # The ceiling this kernel is held against: a pure read of the same number of bytes (packed weight + scales and
        # zeros, 23,953,408 B, rotating through the same number of copies so that it comes from HBM), with every compute
        # unit busy, 1 KB contiguous per wavefront load and all of it requested early; the best of a few shapes of
        # that read.  And an empty kernel of the same grid: what a launch costs inside a graph when it moves nothing.
        probe_bytes = (N * K // 2 + (K // GROUP) * N * 4) // 1024 * 1024
        probe_bufs = [torch.empty(probe_bytes, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(copies)]
        sink = torch.zeros(256, dtype=torch.uint8, device=dev)
        probe = load_probe()
        best = None
        # (the last shape is the column-per-lane pattern of the decode kernel itself: `contiguous` = K / 128, one workgroup per 64 columns)
        for wg, waves, loads, contiguous in ((256, 8, 4, 0), (256, 8, 12, 0), (256, 16, 8, 1), (512, 4, 12, 0), (1, 16, 8, K // 128)):
            def read(i, wg=wg, waves=waves, loads=loads, contiguous=contiguous):
                probe.tpq_probe_read(probe_bufs[i % copies].data_ptr(), probe_bytes, wg, waves, loads, contiguous, sink.data_ptr(), cur())

            gp = graph_of(lambda: [read(i) for i in range(10 * copies)])
            gp.replay(); sync()
            us = steady(gp.replay, sync) / (10 * copies) * 1e3
            if best is None or us < best[0]:
                best = (us, f"column-per-lane pattern, one workgroup of {waves} wavefronts per 64 columns, all loads in flight" if contiguous >= 2 else
                        f"{wg} workgroups x {waves} wavefronts, {loads} KB in flight each, {'contiguous runs' if contiguous else 'interleaved'}")
            del gp
        ge = graph_of(lambda: [probe.tpq_probe_read(None, 0, 256, 8, 4, 0, sink.data_ptr(), cur()) for _ in range(640)])
        ge.replay(); sync()
        extras["empty_kernel_in_graph_us"] = steady(ge.replay, sync) / 640 * 1e3
        extras["int4_gemv_read_ceiling_us"] = best[0]
        extras["int4_gemv_read_ceiling_GBs"] = probe_bytes / (best[0] * 1e-6) / 1e9
        extras["int4_gemv_read_ceiling_pattern"] = best[1]
        extras["int4_gemv_frac_of_read_ceiling"] = best[0] / extras["int4_gemv_us_median_of_7_replays"]
        extras["int4_gemv_steady_frac_of_read_ceiling"] = best[0] / extras["int4_gemv_steady_us"]
        del probe_bufs, ge
        torch.cuda.empty_cache()
    if args.profile_rows > 0:
        mb = args.profile_rows
        xb = torch.from_numpy(rng.normal(0, 1, (mb, K)).astype(np.float32)).to(dev).half()
        yb = torch.empty((mb, N), dtype=torch.float16, device=dev)
        for i in range(200):
            rc = lib.tpq_int4_mm_ws(xb.data_ptr(), _lib.F16, mb, K, packs[i % copies].data_ptr(), 2, N, GROUP,
                                    szs[i % copies].data_ptr(), yb.data_ptr(), ws.data_ptr(), ws.numel(), cur())
            if rc:
                raise RuntimeError(_lib.last_error())
        sync()
        extras["profile_rows"] = mb
    if args.calibrate_copy:
        src_c = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst_c = torch.empty_like(src_c)
        for _ in range(5):
            dst_c.copy_(src_c)  # one elementwise copy kernel: reads 256 MiB, writes 256 MiB
        sync()
        extras["calibration_copy_bytes_each_way"] = 256 << 20
        del src_c, dst_c
    if not args.no_extras:
        # same kernel, launched eagerly through the C ABI (python + launch overhead included)
        sync()
        t = time.perf_counter()
        for i in range(500):
            gemv(i)
        sync()
        extras["int4_gemv_eager_us"] = (time.perf_counter() - t) / 500 * 1e6
        # cache-resident variant: one copy, weights stay in the last-level cache
        gc = graph_of(lambda: [gemv(0) for _ in range(500)])
        gc.replay(); sync()
        ms = steady(gc.replay, sync) / 500
        extras["int4_gemv_cache_resident_us"] = ms * 1e3
        extras["int4_gemv_cache_resident_GBs"] = GEMV_BYTES / (ms * 1e-3) / 1e9
        # batched decode M = 4, 16, 32 (decode kernels) and 256 rows (tiled kernel), rotating weights
        for mb in (4, 16, 32, 256):
            xb = torch.from_numpy(rng.normal(0, 1, (mb, K)).astype(np.float32)).to(dev).half()
            yb = torch.empty((mb, N), dtype=torch.float16, device=dev)

            def gemv_b(i, xb=xb, yb=yb, mb=mb):
                lib.tpq_int4_mm_ws(xb.data_ptr(), _lib.F16, mb, K, packs[i % copies].data_ptr(), 2, N, GROUP,
                                   szs[i % copies].data_ptr(), yb.data_ptr(), ws.data_ptr(), ws.numel(), cur())

            n_b = 260 if mb <= 32 else 64
            gb = graph_of(lambda: [gemv_b(i) for i in range(n_b)])
            gb.replay(); sync()
            ms = steady(gb.replay, sync) / n_b
            if mb >= 128:
                extras[f"int4_gemm_M{mb}_us"] = ms * 1e3
                extras[f"int4_gemm_M{mb}_TFLOPs"] = 2.0 * mb * N * K / (ms * 1e-3) / 1e12
                continue
            bytes_b = N * K // 2 + (K // GROUP) * N * 4 + 2 * mb * K + 2 * mb * N
            extras[f"int4_gemv_M{mb}_us"] = ms * 1e3
            extras[f"int4_gemv_M{mb}_GBs"] = bytes_b / (ms * 1e-3) / 1e9
        # prefill block of 2048 rows on the same weight: the many-row route (dequantise to a dense fp16 weight, then the
        # library's dense tile kernel), both steps through the C ABI, and the dense kernel alone
        mb = 2048
        xb = torch.from_numpy(rng.normal(0, 1, (mb, K)).astype(np.float32)).to(dev).half()
        yb = torch.empty((mb, N), dtype=torch.float16, device=dev)
        dense = torch.empty((N, K), dtype=torch.float16, device=dev)

        def prefill(i, both=True):
            if both:
                lib.tpq_int4_dequantize(packs[i % 4].data_ptr(), 2, N, K, GROUP, szs[i % 4].data_ptr(), _lib.F16, dense.data_ptr(), cur())
            lib.tpq_dense_mm(xb.data_ptr(), _lib.F16, mb, K, dense.data_ptr(), N, yb.data_ptr(), cur())

        for key, both in (("int4_prefill_M2048", True), ("dense_mm_f16_2048x4096x11008", False)):
            gp = graph_of(lambda: [prefill(i, both) for i in range(16)])
            gp.replay(); sync()
            ms = steady(gp.replay, sync) / 16
            extras[key + "_us"] = ms * 1e3
            extras[key + "_TFLOPs"] = 2.0 * mb * N * K / (ms * 1e-3) / 1e12
        del dense, gp
        del packs[1:], szs[1:]
        torch.cuda.empty_cache()
        # 64 and 128 rows on the down-projection shape (11008 -> 4096: 64 workgroups of the tiled kernel per 128 rows): with
        # a workspace the steps of K go to slices whose fp32 sums a second launch adds
        K2, N2 = 11008, 4096
        packs2 = [ops._convert_weight_to_int4pack(torch.randint(0, 16, (N2, K2), dtype=torch.int32, device=dev), 2) for _ in range(12)]
        sz2 = (torch.rand(K2 // GROUP, N2, 2, device=dev) * 0.01).half()
        for mb in (64, 128):
            xb = torch.from_numpy(rng.normal(0, 1, (mb, K2)).astype(np.float32)).to(dev).half()
            yb = torch.empty((mb, N2), dtype=torch.float16, device=dev)
            ws2 = torch.zeros(lib.tpq_int4_mm_rows_workspace_bytes(mb, N2, K2), dtype=torch.uint8, device=dev)

            def mm2(i, xb=xb, yb=yb, mb=mb, ws2=ws2):
                lib.tpq_int4_mm_ws(xb.data_ptr(), _lib.F16, mb, K2, packs2[i % 12].data_ptr(), 2, N2, GROUP, sz2.data_ptr(),
                                   yb.data_ptr(), ws2.data_ptr(), ws2.numel(), cur())

            g2 = graph_of(lambda: [mm2(i) for i in range(48)])
            g2.replay(); sync()
            ms = steady(g2.replay, sync) / 48
            extras[f"int4_mm_M{mb}_11008x4096_us"] = ms * 1e3
            extras[f"int4_mm_M{mb}_11008x4096_TFLOPs"] = 2.0 * mb * N2 * K2 / (ms * 1e-3) / 1e12
        del packs2, g2
        torch.cuda.empty_cache()
        # int8 weight-only decode (next-row op _weight_int8pack_mm): same shape, one byte per weight
        w8s = [torch.randint(-128, 128, (N, K), dtype=torch.int8, device=dev) for _ in range(14)]  # 631 MB
        s8 = torch.rand(N, device=dev) * 0.01
        for mb in (1, 8, 32):
            xb = torch.from_numpy(rng.normal(0, 1, (mb, K)).astype(np.float32)).to(dev).half()
            yb = torch.empty((mb, N), dtype=torch.float16, device=dev)

            def i8mm(i, xb=xb, yb=yb, mb=mb):
                lib.tpq_weight_int8pack_mm(xb.data_ptr(), _lib.F16, mb, K, w8s[i % 14].data_ptr(), s8.data_ptr(), N,
                                           yb.data_ptr(), cur())

            g8 = graph_of(lambda: [i8mm(i) for i in range(140)])
            g8.replay(); sync()
            ms = steady(g8.replay, sync) / 140
            extras[f"int8pack_M{mb}_us"] = ms * 1e3
            extras[f"int8pack_M{mb}_GBs"] = (N * K + 4 * N + 2 * mb * K + 2 * mb * N) / (ms * 1e-3) / 1e9
        del w8s
        torch.cuda.empty_cache()
        # packed n-bit weight-only decode (int2 / intx / binary modules): same shape, bits per weight in
        # {1, 2, 4, 8}, float32 (scale, zero) per group of 128; enough rotating copies to stream from HBM
        G = K // 128
        szf = torch.stack([torch.rand(G, N, device=dev) * 0.01, torch.full((G, N), 2.0, device=dev)], dim=-1).contiguous()
        for bits in (1, 2, 4, 8):
            row_bytes = K * bits // 8
            n_copies = max(2, min(60, (600 << 20) // (N * row_bytes)))
            wl = [torch.randint(0, 256, (N, row_bytes), dtype=torch.uint8, device=dev) for _ in range(n_copies)]
            for mb in (1, 8):  # one row: the row kernel; eight: the matrix-core kernel
                xb = torch.from_numpy(rng.normal(0, 1, (mb, K)).astype(np.float32)).to(dev).half()
                yb = torch.empty((mb, N), dtype=torch.float16, device=dev)

                def lbmm(i, wl=wl, bits=bits, n_copies=n_copies, xb=xb, yb=yb, mb=mb):
                    lib.tpq_lowbit_mm(xb.data_ptr(), _lib.F16, mb, K, wl[i % n_copies].data_ptr(), bits, 0, N, 128,
                                      szf.data_ptr(), None, yb.data_ptr(), cur())

                gl = graph_of(lambda: [lbmm(i) for i in range(2 * n_copies)])
                gl.replay(); sync()
                ms = steady(gl.replay, sync) / (2 * n_copies)
                extras[f"lowbit{bits}_M{mb}_us"] = ms * 1e3
                extras[f"lowbit{bits}_M{mb}_GBs"] = (N * row_bytes + 8 * G * N + 2 * mb * K + 2 * mb * N) / (ms * 1e-3) / 1e9
            del wl
        torch.cuda.empty_cache()

    if not args.no_extras and not args.gemv_only:
        # int8 prefill GEMM with fused dequant: M=2048, K=4096, N=4096, bf16 in/out
        M8, K8, N8 = 2048, 4096, 4096
        xa = rng.normal(0, 1, (M8, K8)).astype(np.float32)
        xa[:, rng.choice(K8, 41, replace=False)] *= 20.0
        xa_d = torch.from_numpy(xa).to(dev).bfloat16()
        w8_d = torch.from_numpy(rng.normal(0, 0.02, (N8, K8)).astype(np.float32)).to(dev).bfloat16()
        a_q, a_s = ops._quantize_int8_rowwise(xa_d, 1e-5)
        w_q, w_s = ops._quantize_int8_rowwise(w8_d, 1e-5)
        out8 = torch.empty((M8, N8), dtype=torch.bfloat16, device=dev)

        def gemm8():
            lib.tpq_int8_mm_dequant(a_q.data_ptr(), w_q.data_ptr(), a_s.data_ptr(), w_s.data_ptr(), None,
                                    out8.data_ptr(), _lib.BF16, M8, N8, K8, cur())

        # warm-up of at least 30 ms, then the median of 7 batches of 50 launches (the first batches after the
        # host-side set-up above run 10..30 % slower)
        ms = steady(gemm8, sync, 50)
        tops = 2.0 * M8 * N8 * K8 / (ms * 1e-3) / 1e12
        extras["int8_gemm_2048x4096x4096_us"] = ms * 1e3
        extras["int8_gemm_TOPS"] = tops
        extras["int8_gemm_frac_of_mfma_peak"] = tops / INT8_PEAK_TOPS
        roofline_int8 = {"bound": "mfma", "achieved": round(tops, 1), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                         "frac": round(tops / INT8_PEAK_TOPS, 4), "traffic": measured_traffic_bytes(INT8_PROFILE),
                         "kernel": "gemm_stagger_kernel<bf16 dequant epilogue, int8> (tpq_int8_mm_dequant)",
                         "algorithmic_ops_per_launch": 2 * M8 * N8 * K8, "avg_launch_us": ms * 1e3,
                         "workload": "int8 x int8 prefill GEMM M=2048 K=4096 N=4096, fused per-row x per-channel dequant, bf16 out (BASELINE configs[2])"}
        # the vendor library's int8 GEMM on the same operands (torch._int_mm -> hipBLASLt), for scale: it
        # writes raw int32 sums, without the dequant epilogue that the kernel above includes
        try:
            w_qt = w_q.t()
            ms_lib = steady(lambda: torch._int_mm(a_q, w_qt), sync, 50)
            extras["int8_gemm_vendor_int_mm_us"] = ms_lib * 1e3
            extras["int8_gemm_vendor_int_mm_TOPS"] = 2.0 * M8 * N8 * K8 / (ms_lib * 1e-3) / 1e12
        except Exception as exc:  # the library may lack the shape: a comparison figure only
            extras["int8_gemm_vendor_int_mm_us"] = None
            extras["int8_gemm_vendor_note"] = str(exc)[:80]
        acc_chk = (a_q[:64].double() @ w_q.double().t())
        fused_chk = ((acc_chk.float() * a_s[:64, None]) * w_s[None, :]).bfloat16()
        extras["int8_gemm_rows_checked_equal"] = bool(torch.equal(fused_chk, out8[:64]))

        # the same product for decode batches and short prompts (1 / 16 / 128 rows): the row kernel, the decode kernel, and the tiled
        # kernel with its k range in slices (workspace entry point), weights rotating through 30 copies (0.5 GB)
        w_rot = [w_q.clone() for _ in range(30)]
        for m_small in (1, 16, 128):
            a_small, s_small = a_q[:m_small].contiguous(), a_s[:m_small].contiguous()
            out_small = torch.empty((m_small, N8), dtype=torch.bfloat16, device=dev)
            ws_bytes = int(lib.tpq_int8_mm_workspace_bytes(m_small, N8, K8))
            scratch = torch.empty(max(ws_bytes, 16) // 4, dtype=torch.int32, device=dev)

            def gemm_small(i, a_small=a_small, s_small=s_small, out_small=out_small, m_small=m_small, scratch=scratch, ws_bytes=ws_bytes):
                lib.tpq_int8_mm_dequant_ws(a_small.data_ptr(), w_rot[i % 30].data_ptr(), s_small.data_ptr(), w_s.data_ptr(), None,
                                           out_small.data_ptr(), _lib.BF16, m_small, N8, K8, scratch.data_ptr(), ws_bytes, cur())

            gemm_small(0); sync()
            gs8 = graph_of(lambda: [gemm_small(i) for i in range(120)])
            gs8.replay(); sync()
            ms = steady(gs8.replay, sync) / 120
            extras[f"int8_gemm_{m_small}x4096x4096_us"] = ms * 1e3
            extras[f"int8_gemm_{m_small}x4096x4096_weight_GBs"] = N8 * K8 / (ms * 1e-3) / 1e9
            extras[f"int8_gemm_{m_small}_rows_equal_big_gemm"] = bool(torch.equal(out_small, out8[:m_small]))
        del w_rot

        # activation quantizer on the same activations: 2*M*K + M*K + 4*M bytes
        cq = torch.empty((M8, K8), dtype=torch.int8, device=dev)
        sq = torch.empty((M8,), dtype=torch.float32, device=dev)

        def quant():
            lib.tpq_quantize_rowwise(xa_d.data_ptr(), _lib.BF16, M8, K8, 1e-5, 127.0, -127, 127, 0, cq.data_ptr(),
                                     sq.data_ptr(), cur())

        for _ in range(5):
            quant()
        ms = steady(quant, sync, 100)
        extras["quantize_2048x4096_bf16_us"] = ms * 1e3
        extras["quantize_GBs"] = (3 * M8 * K8 + 4 * M8) / (ms * 1e-3) / 1e9
        # the same with the input rotating through 24 copies (403 MB: beyond the 256 MB memory-side cache), i.e. read
        # from HBM every time; the figure above re-reads one 16.8 MB input, as a quantizer behind the kernel that
        # produced its input does
        xa_rot = [xa_d] + [xa_d.clone() for _ in range(23)]
        turn = [0]

        def quant_rot():
            turn[0] = (turn[0] + 1) % 24
            lib.tpq_quantize_rowwise(xa_rot[turn[0]].data_ptr(), _lib.BF16, M8, K8, 1e-5, 127.0, -127, 127, 0, cq.data_ptr(),
                                     sq.data_ptr(), cur())

        ms = steady(quant_rot, sync, 96)
        extras["quantize_2048x4096_bf16_hbm_rotated_us"] = ms * 1e3
        extras["quantize_hbm_rotated_GBs"] = (3 * M8 * K8 + 4 * M8) / (ms * 1e-3) / 1e9

        # rms_norm of the same prefill block (the stand-alone op; at decode sizes the norm is folded into the int4 launches):
        # 2*M*K read + 2*M*K written + 2*K bytes
        gn = (torch.rand(K8, device=dev) + 0.5).to(torch.bfloat16)
        yn = torch.empty_like(xa_d)

        def norm():
            lib.tpq_rms_norm(xa_d.data_ptr(), _lib.BF16, M8, K8, gn.data_ptr(), 1e-5, yn.data_ptr(), cur())

        for _ in range(5):
            norm()
        ms = steady(norm, sync, 100)
        extras["rms_norm_2048x4096_bf16_us"] = ms * 1e3
        extras["rms_norm_GBs"] = (4 * M8 * K8 + 2 * K8) / (ms * 1e-3) / 1e9

        def norm_rot():
            turn[0] = (turn[0] + 1) % 24
            lib.tpq_rms_norm(xa_rot[turn[0]].data_ptr(), _lib.BF16, M8, K8, gn.data_ptr(), 1e-5, yn.data_ptr(), cur())

        ms = steady(norm_rot, sync, 96)
        extras["rms_norm_2048x4096_bf16_hbm_rotated_us"] = ms * 1e3
        extras["rms_norm_hbm_rotated_GBs"] = (4 * M8 * K8 + 2 * K8) / (ms * 1e-3) / 1e9
        del xa_rot

        # block-wise affine quantizer: the same activations in f32, one block per row -> int8 (4 + 1 bytes per
        # element), and a 4096 x 4096 f32 weight in groups of 128 -> packed 4-bit (4 + 0.5) and back (0.5 + 4)
        import ctypes
        xa32 = xa_d.float()
        shape2 = (ctypes.c_int64 * 2)(M8, K8)
        row_block = (ctypes.c_int64 * 2)(1, K8)
        shape_p, row_block_p = ctypes.cast(shape2, ctypes.c_void_p), ctypes.cast(row_block, ctypes.c_void_p)

        def affine_rows():
            lib.tpq_quantize_affine(xa32.data_ptr(), _lib.F32, 2, shape_p, row_block_p, a_s.data_ptr(), M8, None, 0,
                                    _lib.STORAGE_I8, -127, 127, cq.data_ptr(), cur())

        for _ in range(5):
            affine_rows()
        ms = steady(affine_rows, sync, 100)
        extras["quantize_affine_2048x4096_rows_int8_us"] = ms * 1e3
        extras["quantize_affine_rows_GBs"] = (5 * M8 * K8 + 4 * M8) / (ms * 1e-3) / 1e9
        wf = torch.from_numpy(rng.normal(0, 0.02, (4096, 4096)).astype(np.float32)).to(dev)
        gs = (wf.view(4096, 32, 128).abs().amax(dim=2) / 7.0).reshape(-1).contiguous()
        gz = torch.full_like(gs, 8.0)
        w4 = torch.empty((4096 * 4096 // 2,), dtype=torch.uint8, device=dev)
        wback = torch.empty_like(wf)
        shape_w = (ctypes.c_int64 * 2)(4096, 4096)
        grp_block = (ctypes.c_int64 * 2)(1, 128)
        shape_wp, grp_block_p = ctypes.cast(shape_w, ctypes.c_void_p), ctypes.cast(grp_block, ctypes.c_void_p)

        def affine_q4():
            lib.tpq_quantize_affine(wf.data_ptr(), _lib.F32, 2, shape_wp, grp_block_p, gs.data_ptr(), gs.numel(),
                                    gz.data_ptr(), gz.numel(), _lib.STORAGE_U4X2, 0, 15, w4.data_ptr(), cur())

        def affine_dq4():
            lib.tpq_dequantize_affine(w4.data_ptr(), _lib.STORAGE_U4X2, 2, shape_wp, grp_block_p, gs.data_ptr(), gs.numel(),
                                      gz.data_ptr(), gz.numel(), wback.data_ptr(), cur())

        for fn, key in ((affine_q4, "quantize_affine_4096x4096_g128_u4"), (affine_dq4, "dequantize_affine_4096x4096_g128_u4")):
            for _ in range(5):
                fn()
            ms = steady(fn, sync, 100)
            extras[key + "_us"] = ms * 1e3
            extras[key + "_GBs"] = (4.5 * 4096 * 4096 + 8 * gs.numel()) / (ms * 1e-3) / 1e9

        # BitNet ternary: M in {1,128}, 2560 -> 6912 and 6912 -> 2560 (weights cache resident at this size)
        for (mt, kt, nt) in ((1, 2560, 6912), (1, 6912, 2560), (8, 2560, 6912), (8, 6912, 2560), (128, 2560, 6912), (128, 6912, 2560)):
            tern = rng.choice(np.int8([-1, 0, 1]), size=(nt, kt), p=[0.325, 0.35, 0.325])
            pk = ops.pack_ternary(torch.from_numpy(tern).to(dev))
            xt = torch.from_numpy(rng.normal(0, 1, (mt, kt)).astype(np.float32)).to(dev)
            xq_t, rs_t = ops._quantize_int8_rowwise(xt, 1e-5)
            yt = torch.empty((mt, nt), dtype=torch.float16, device=dev)

            # (the scratch matrix for the split-K partial sums, as the op wrapper passes it; 0 bytes for most shapes)
            tws_bytes = int(lib.tpq_ternary_mm_workspace_bytes(mt, nt, kt))
            tws = torch.empty(max(tws_bytes, 4) // 4, dtype=torch.int32, device=dev)

            def tmm(xq_t=xq_t, rs_t=rs_t, pk=pk, yt=yt, mt=mt, kt=kt, nt=nt, tws=tws, tws_bytes=tws_bytes):
                lib.tpq_ternary_mm_ws(xq_t.data_ptr(), rs_t.data_ptr(), pk.data_ptr(), 0.0173, None, mt, nt, kt,
                                      yt.data_ptr(), _lib.F16, None, tws.data_ptr(), tws_bytes, cur())

            gt = graph_of(lambda: [tmm() for _ in range(200)])
            gt.replay(); sync()
            ms = steady(gt.replay, sync) / 200
            key = f"ternary_M{mt}_{kt}x{nt}"
            extras[key + "_us"] = ms * 1e3
            if mt <= 8:
                t_bytes = nt * kt // 4 + mt * kt + 4 * mt + 2 * mt * nt
                extras[key + "_GBs_cache_resident"] = t_bytes / (ms * 1e-3) / 1e9
                if mt == 1:  # the same call on 160 rotating copies of the packed weight (0.7 GB): streamed from HBM
                    pks = [pk] + [pk.clone() for _ in range(159)]

                    def tmm_rot(i, pks=pks, xq_t=xq_t, rs_t=rs_t, yt=yt, mt=mt, kt=kt, nt=nt):
                        lib.tpq_ternary_mm(xq_t.data_ptr(), rs_t.data_ptr(), pks[i % 160].data_ptr(), 0.0173, None, mt, nt, kt,
                                           yt.data_ptr(), _lib.F16, None, cur())

                    gr = graph_of(lambda: [tmm_rot(i) for i in range(480)])
                    gr.replay(); sync()
                    ms_rot = steady(gr.replay, sync) / 480
                    extras[key + "_hbm_rotated_us"] = ms_rot * 1e3
                    extras[key + "_GBs_hbm_rotated"] = t_bytes / (ms_rot * 1e-3) / 1e9
                    del pks, gr
            else:
                extras[key + "_TOPS"] = 2.0 * mt * nt * kt / (ms * 1e-3) / 1e12

    if not args.no_extras and not args.gemv_only and not args.no_layer:
        del packs, szs
        torch.cuda.empty_cache()
        extras.update(decoder_layer_share(dev))

    line = {
        "metric": METRIC,
        "value": round(gbs, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "int4 weight-only decode GEMV M=1 K=4096 N=11008 group=128 fp16 (BASELINE configs[1])",
            "weights": f"reference device int4 layout, {copies} rotating copies (HBM resident, not cache resident)",
            "launch": "K steps in one HIP graph replay",
        },
        "roofline": {
            "bound": "hbm",
            "achieved": round(gbs, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4),
            "traffic": measured_traffic_bytes(),
            "kernel": "int4_decode_kernel<f16, M=1, g=128>",
            "algorithmic_bytes_per_launch": GEMV_BYTES,
            "avg_launch_us": ms_per_step * 1e3,
        },
        "roofline_int8": roofline_int8,
        "cpu_baseline": None,
        "extras": {k: (round(v, 4) if isinstance(v, float) else v) for k, v in extras.items()},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(x16, codes, sz16, want)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
