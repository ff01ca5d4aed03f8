"""GPU parity: ternary pack/unpack (bit-exact) and the BitNet packed matmul (exact int32 sums,
fp32 outputs equal to the oracle's evaluation of the reference formula)."""
import itertools

import numpy as np
import pytest
import torch

import oracle
from gpu_util import DEV, TORCH_DT, dev, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from tensorplay_amd import ops as _ops

    return _ops


def _ternary(rng, shape):
    return rng.choice(np.int8([-1, 0, 1]), size=shape, p=[0.325, 0.35, 0.325])


@pytest.mark.parametrize("shape", [(2, 9), (1, 1), (7, 4), (6912, 2560), (33, 1023), (3, 5, 10)])
def test_pack_unpack_bit_exact(ops, shape):
    rng = np.random.default_rng(sum(shape))
    codes = _ternary(rng, shape)
    want = oracle.pack_ternary(codes)
    got = ops.pack_ternary(dev(codes))
    assert got.dtype == torch.uint8 and tuple(got.shape) == want.shape
    np.testing.assert_array_equal(host(got), want)
    back = ops.unpack_ternary(got, shape[-1])
    np.testing.assert_array_equal(host(back), codes)


def test_unpack_every_byte_value(ops):
    every = np.arange(256, dtype=np.uint8).reshape(256, 1)
    np.testing.assert_array_equal(host(ops.unpack_ternary(dev(every), 4)), oracle.unpack_ternary(every, 4))
    table = np.int8(list(itertools.product([-1, 0, 1], repeat=4)))
    np.testing.assert_array_equal(host(ops.pack_ternary(dev(table))), oracle.pack_ternary(table))


# (M, K, N): decode kernel, matrix-core kernel, generic kernel
CASES = [(1, 2560, 6912), (1, 6912, 2560), (4, 2560, 256), (8, 128, 67), (5, 64, 9), (128, 2560, 6912),
         (128, 6912, 2560), (16, 256, 100), (33, 48, 70), (3, 9, 5), (2, 10, 4), (9, 2560, 130),
         (200, 512, 70), (97, 256, 33), (300, 256, 64),
         # tile kernel below nine rows (many / few tiles of 32 channels) and beyond 256 rows
         (4, 256, 4200), (7, 512, 72), (8, 768, 40), (513, 512, 100), (700, 256, 4160),
         # matrix-core decode kernel: each workgroup shape (by N), ragged N, one and two slabs of rows
         (1, 4096, 4100), (2, 2560, 8200), (16, 512, 8192), (3, 1024, 11010), (15, 256, 16390), (17, 768, 50),
         (32, 512, 8208), (31, 6912, 2560), (12, 256, 1), (1, 256, 17), (64, 512, 100), (49, 256, 8200), (63, 768, 16400),
         # long K against at most 256 blocks of 16 channels: 16 wavefronts per workgroup (1, 2, 4 activation loads, two slabs)
         (3, 6144, 4096), (8, 6912, 2560), (16, 8192, 1048), (23, 7168, 520),
         # slab kernel (33 rows and more, K % 128 == 0): one unit, ragged rows and channels, 21 units = two splits,
         # 40 units = two full splits, three splits with a short last one
         (33, 128, 8), (40, 384, 136), (129, 2688, 200), (128, 5120, 264), (70, 5248, 130),
         # two splits are taken up to 64 rows: 21 units (a short second split), 32 units, 40 units; above 64 rows from
         # 32 units on (24 units at 97 rows go to the tile kernel)
         (40, 2688, 200), (64, 4096, 520), (33, 5120, 136), (97, 4096, 520), (128, 4224, 136), (97, 3072, 264)]


@pytest.mark.parametrize("M,K,N", CASES)
def test_ternary_mm_exact(ops, M, K, N):
    rng = np.random.default_rng(M + K + N)
    codes = _ternary(rng, (N, K))
    packed = oracle.pack_ternary(codes)
    x = rng.normal(size=(M, K)).astype(np.float32)
    xq, rs = oracle.quantize_int8_rowwise(x, "f32", 1e-5)
    w_scale = float(np.float16(0.0173))   # an fp16-representable absmean scale, applied in fp32
    bias = rng.normal(0, 0.01, N).astype(np.float32)
    want, want_acc = oracle.ternary_mm(xq, rs, packed, w_scale, K, bias=bias)
    got, acc = ops.ternary_mm(dev(xq), dev(rs), dev(packed), w_scale, K, bias=dev(bias), return_acc=True)
    np.testing.assert_array_equal(host(acc), want_acc)
    np.testing.assert_array_equal(want_acc, xq.astype(np.int32) @ codes.astype(np.int32).T)
    np.testing.assert_array_equal(host(got), want)
    for dt in ("f16", "bf16"):
        w16, _ = oracle.ternary_mm(xq, rs, packed, w_scale, K, out_dtype=dt)
        g16 = ops.ternary_mm(dev(xq), dev(rs), dev(packed), w_scale, K, out_dtype=TORCH_DT[dt])
        np.testing.assert_array_equal(host(g16), w16)


@pytest.mark.parametrize("M,K,N", [(16, 2560, 6912), (32, 6912, 2560), (8, 8192, 28672)])
def test_ternary_decode_kernel_at_model_sizes(ops, M, K, N):
    """The matrix-core decode kernel at real layer sizes, any byte value in the packed weight: exact accumulators,
    and linear in the activations (x and -x give opposite sums)."""
    rng = np.random.default_rng(M + K + N)
    packed = rng.integers(0, 256, size=(N, K // 4)).astype(np.uint8)
    x = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
    rs = np.ones(M, np.float32)
    _, want_acc = oracle.ternary_mm(x, rs, packed, 1.0, K)
    _, acc = ops.ternary_mm(dev(x), dev(rs), dev(packed), 1.0, K, return_acc=True)
    np.testing.assert_array_equal(host(acc), want_acc)
    _, neg = ops.ternary_mm(dev((-x).astype(np.int8)), dev(rs), dev(packed), 1.0, K, return_acc=True)
    assert torch.equal(neg, -acc)


def test_ternary_mm_arbitrary_bytes_and_extremes(ops):
    """Any byte is a legal packed value (0b10 decodes to -2); activations at the int8 extremes."""
    rng = np.random.default_rng(8)
    K, N = 6912, 64
    packed = rng.integers(0, 256, size=(N, K // 4)).astype(np.uint8)
    x = np.where(rng.random((3, K)) < 0.5, -127, 127).astype(np.int8)
    rs = np.ones(3, np.float32)
    want, want_acc = oracle.ternary_mm(x, rs, packed, 1.0, K)
    got, acc = ops.ternary_mm(dev(x), dev(rs), dev(packed), 1.0, K, return_acc=True)
    np.testing.assert_array_equal(host(acc), want_acc)
    x128 = np.repeat(x, 43, axis=0)[:128]
    _, want_acc = oracle.ternary_mm(x128, np.ones(128, np.float32), packed, 1.0, K)
    _, acc = ops.ternary_mm(dev(x128), dev(np.ones(128, np.float32)), dev(packed), 1.0, K, return_acc=True)
    np.testing.assert_array_equal(host(acc), want_acc)


@pytest.mark.parametrize("M,K,N", [(128, 2560, 200), (40, 2560, 130), (64, 4096, 264), (96, 1152, 72)])
def test_ternary_slab_arbitrary_bytes(ops, M, K, N):
    """The slab kernel (33 rows and more) with any byte value in the packed weight (0b10 decodes to -2) and the
    activations at the int8 extremes, one and two splits of K, channel counts that are and are not multiples of four:
    exact accumulators, and the scaled output equal to the oracle's."""
    rng = np.random.default_rng(M + K + N)
    packed = rng.integers(0, 256, size=(N, K // 4)).astype(np.uint8)
    x = np.where(rng.random((M, K)) < 0.5, -127, 127).astype(np.int8)
    x[1::3] = rng.integers(-127, 128, size=x[1::3].shape).astype(np.int8)
    rs = (rng.random(M) * 0.01 + 1e-3).astype(np.float32)
    want, want_acc = oracle.ternary_mm(x, rs, packed, 0.03, K)
    got, acc = ops.ternary_mm(dev(x), dev(rs), dev(packed), 0.03, K, return_acc=True)
    np.testing.assert_array_equal(host(acc), want_acc)
    np.testing.assert_array_equal(host(got), want)
    got_only = ops.ternary_mm(dev(x), dev(rs), dev(packed), 0.03, K)
    np.testing.assert_array_equal(host(got_only), want)


@pytest.mark.parametrize("K,N", [(64, 3), (64, 5), (64, 70001), (128, 262144), (192, 1000), (320, 77), (1024, 1), (2560, 6912), (6912, 2560), (4096, 4100),
                                 (8192, 4096), (5120, 5120), (2048, 259), (8192, 28672), (4096, 32000)])
def test_ternary_one_row_kernel_arbitrary_bytes(ops, K, N):
    """One activation row on up to 8 MB of packed weights takes the flat dot-product kernel (one 16-byte chunk per
    thread, the channel sums added up in LDS): any byte value in the packed weight (0b10 decodes to -2), activations
    over the whole int8 range with -128 and the extremes in it, K % 64 == 0 only, channel counts that leave the last
    workgroup short: exact accumulators, the scaled output with and without bias equal to the oracle's in every
    output type, and linear in the activations."""
    rng = np.random.default_rng(K + N)
    packed = rng.integers(0, 256, size=(N, K // 4)).astype(np.uint8)
    x = rng.integers(-128, 128, size=(1, K)).astype(np.int8)
    x[0, ::7] = np.where(rng.random(x[0, ::7].shape) < 0.5, -127, 127)
    rs = np.float32([0.0071])
    bias = rng.normal(0, 0.05, N).astype(np.float32)
    want, want_acc = oracle.ternary_mm(x, rs, packed, 0.03, K, bias=bias)
    got, acc = ops.ternary_mm(dev(x), dev(rs), dev(packed), 0.03, K, bias=dev(bias), return_acc=True)
    np.testing.assert_array_equal(host(acc), want_acc)
    np.testing.assert_array_equal(host(got), want)
    for dt in ("f16", "bf16"):
        w16, _ = oracle.ternary_mm(x, rs, packed, 0.03, K, out_dtype=dt)
        g16 = ops.ternary_mm(dev(x), dev(rs), dev(packed), 0.03, K, out_dtype=TORCH_DT[dt])
        np.testing.assert_array_equal(host(g16), w16)
    flipped = np.clip(-x.astype(np.int32), -127, 127).astype(np.int8)
    _, want_neg = oracle.ternary_mm(flipped, rs, packed, 0.03, K)
    _, neg = ops.ternary_mm(dev(flipped), dev(rs), dev(packed), 0.03, K, return_acc=True)
    np.testing.assert_array_equal(host(neg), want_neg)
