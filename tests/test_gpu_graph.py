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
