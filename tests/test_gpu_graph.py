"""The ops of the path recorded into one HIP graph and replayed: every replay must give the bits of the eager call on
the same inputs.  The library issues no memory set, no allocation and no synchronization of its own, so a launch
sequence is capturable as it is; the replays are separated by eager work and synchronizations, and the inputs change
between them (a node that kept a stale pointer or a counter that was not put back would show on the second replay)."""
import numpy as np
import pytest
import torch

from gpu_util import DEV

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from tensorplay_amd import ops as _ops

    return _ops


def _int4_weight(ops, rng, n, k):
    codes = torch.from_numpy(rng.integers(0, 16, (n, k)).astype(np.int32)).to(DEV)
    sz = (torch.rand(k // 128, n, 2, device=DEV) * 0.02 - 0.01).half()
    return ops._convert_weight_to_int4pack(codes, 2), sz


def test_replays_equal_eager(ops):
    rng = np.random.default_rng(0)
    torch.manual_seed(0)
    k = 4096
    wq, szq = _int4_weight(ops, rng, 1024, k)
    wk, szk = _int4_weight(ops, rng, 256, k)
    wg, szg = _int4_weight(ops, rng, 1408, k)
    wu, szu = _int4_weight(ops, rng, 1408, k)
    wd, szd = _int4_weight(ops, rng, 4096, 1408 - 1408 % 128)
    g1 = (torch.rand(k, device=DEV) + 0.5).half()
    w8 = torch.randint(-127, 128, (512, k), dtype=torch.int8, device=DEV)
    cs = torch.rand(512, device=DEV) * 0.01
    tern = torch.from_numpy(rng.choice([-1, 0, 1], size=(2560, 6912), p=[0.325, 0.35, 0.325]).astype(np.int8)).to(DEV)
    tpacked = ops.pack_ternary(tern)

    x1 = torch.empty(1, k, device=DEV, dtype=torch.float16)     # one row: the column-per-lane kernel
    x8 = torch.empty(8, k, device=DEV, dtype=torch.float16)     # a decode batch: the all-in-flight kernel and its fusions
    xb = torch.empty(160, k, device=DEV, dtype=torch.bfloat16)  # a prefill block: quantizer, sliced int8 product
    xt = torch.empty(128, 6912, device=DEV, dtype=torch.bfloat16)

    def fill(seed):
        gen = torch.Generator(device=DEV).manual_seed(seed)
        for t in (x1, x8, xb, xt):
            t.copy_(torch.randn(t.shape, device=DEV, generator=gen).to(t.dtype))

    def sequence():
        out = [ops._weight_int4pack_mm(x1, wq, 128, szq)]
        out += ops.int4pack_mm_multi(x8, [wq, wk], 128, [szq, szk], norm_weight=g1, eps=1e-5)
        h = ops.int4pack_mm_swiglu(x8, wg, wu, 128, szg, szu, norm_weight=g1, eps=1e-5)
        out.append(h)
        out.append(ops.int4pack_mm_add(h[:, :wd.shape[1] * 32].contiguous(), wd, 128, szd, x8))
        out.append(ops.rms_norm(xb, None, 1e-5))
        codes, scales = ops._quantize_int8_rowwise(xb, 1e-5)
        out += [codes, scales, ops.int8_mm_dequant(codes, w8, scales, cs, None, torch.bfloat16)]
        tc, ts = ops._quantize_int8_rowwise(xt, 1e-5)
        out.append(ops.ternary_mm(tc, ts, tpacked, 0.02, 6912, None, torch.bfloat16))
        return out

    fill(1)
    sequence()  # warm-up outside the capture: workspaces the wrappers keep are created here
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            recorded = sequence()
    torch.cuda.synchronize()
    for seed in (2, 3, 4):
        fill(seed)
        want = [t.clone() for t in sequence()]       # eager, same inputs
        torch.cuda.synchronize()
        for t in recorded:
            t.fill_(0)                                # eager work between the replays; stale results cannot pass
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for idx, (got, ref) in enumerate(zip(recorded, want)):
            assert torch.equal(got, ref), f"replay with seed {seed}: output {idx} differs from the eager call"


def test_noalloc_entry_point_under_capture():
    """tpq_int8_mm_dequant_noalloc recorded into graphs.  The first graph holds what is (when this file runs in a fresh
    process) the first call on this device, so the lookup of the built-in buffer's address happens during the capture;
    the second is recorded after eager calls.  Between the replays the inputs change and a smaller eager call leaves its
    partial sums in the shared buffer.  Every replay must equal tpq_int8_mm_dequant_ws with a caller's workspace, bit
    for bit (both add the same exact int32 partial sums)."""
    import ctypes

    from tensorplay_amd import _lib

    lib = _lib.load()

    def ptr(t):
        return ctypes.c_void_p(t.data_ptr()) if t is not None else None

    M, N, K = 300, 264, 8192   # few tiles, long K: the shape is one that cuts the k range into slices
    need = lib.tpq_int8_mm_workspace_bytes(M, N, K)
    assert 0 < need <= lib.tpq_int8_mm_noalloc_max_bytes()
    a = torch.empty((M, K), dtype=torch.int8, device=DEV)
    w = torch.empty((N, K), dtype=torch.int8, device=DEV)
    rs = torch.empty(M, device=DEV)
    cs = torch.empty(N, device=DEV)
    bias = torch.empty(N, device=DEV)
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    # the smaller problem that dirties the shared buffer between replays
    m2, n2, k2 = 130, 200, 4096
    assert lib.tpq_int8_mm_workspace_bytes(m2, n2, k2) > 0
    a2 = torch.randint(-128, 128, (m2, k2), dtype=torch.int8, device=DEV)
    w2 = torch.randint(-128, 128, (n2, k2), dtype=torch.int8, device=DEV)
    rs2, cs2 = torch.rand(m2, device=DEV), torch.rand(n2, device=DEV)
    out2 = torch.empty((m2, n2), dtype=torch.float32, device=DEV)

    def fill(seed):
        gen = torch.Generator(device=DEV).manual_seed(seed)
        a.copy_(torch.randint(-128, 128, a.shape, device=DEV, generator=gen).to(torch.int8))
        w.copy_(torch.randint(-128, 128, w.shape, device=DEV, generator=gen).to(torch.int8))
        rs.copy_(torch.rand(M, device=DEV, generator=gen) * 0.02 + 0.001)
        cs.copy_(torch.rand(N, device=DEV, generator=gen) * 0.002 + 0.0001)
        bias.copy_(torch.randn(N, device=DEV, generator=gen) * 0.01)

    def record(out, dt):
        stream = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            with torch.cuda.graph(graph, stream=stream):
                s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
                rc = lib.tpq_int8_mm_dequant_noalloc(ptr(a), ptr(w), ptr(rs), ptr(cs), ptr(bias), ptr(out), dt, M, N, K, s)
        assert rc == 0, _lib.last_error()
        torch.cuda.synchronize()
        return graph

    def check(graph, out, dt, seeds):
        for seed in seeds:
            fill(seed)
            s = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            want = torch.full_like(out, 5)
            rc = lib.tpq_int8_mm_dequant_ws(ptr(a), ptr(w), ptr(rs), ptr(cs), ptr(bias), ptr(want), dt, M, N, K, ptr(ws), need, s)
            assert rc == 0, _lib.last_error()
            # an eager call on a smaller problem: its partial sums stay in the shared buffer
            assert lib.tpq_int8_mm_dequant_noalloc(ptr(a2), ptr(w2), ptr(rs2), ptr(cs2), None, ptr(out2), 0, m2, n2, k2, s) == 0
            out.fill_(3)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out.view(torch.uint8), want.view(torch.uint8)), f"replay with seed {seed} differs from the _ws call"

    fill(10)
    out32 = torch.empty((M, N), dtype=torch.float32, device=DEV)
    first = record(out32, 0)            # no noalloc call has been made before this capture in this file
    check(first, out32, 0, (11, 12, 13))
    out16 = torch.empty((M, N), dtype=torch.bfloat16, device=DEV)
    second = record(out16, 2)           # recorded after eager calls
    check(second, out16, 2, (14, 15))
    check(first, out32, 0, (16,))       # and the first graph still replays correctly
