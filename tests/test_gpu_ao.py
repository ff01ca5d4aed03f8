"""The ao modules on the GPU against the CPU oracle and the reference tests' closed forms
(test/quantization/test_int4_modules.py:26-82, test_awq.py:75-99, test_int8_mixed_precision.py:26-34,
219-229, test_native_1bit.py:200-210)."""
import numpy as np
import pytest
import torch
import torch.nn as nn

import oracle
from gpu_util import DEV, assert_close_norm, dev, host
from helpers import bits_of, cast_bits

pytestmark = pytest.mark.gpu


def _ao():
    import tensorplay_amd.ao.quantization as q
    return q


@pytest.mark.parametrize("dtype,tag", [(torch.float16, "f16"), (torch.bfloat16, "bf16"), (torch.float32, "f32")])
@pytest.mark.parametrize("rows", [1, 8, 33])
def test_weight_only_int4_linear(dtype, tag, rows):
    q = _ao()
    rng = np.random.default_rng(31)
    N, K, g = 264, 512, 128
    lin = nn.Linear(K, N, bias=True)
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy(rng.normal(0, 0.02, (N, K)).astype(np.float32)))
        lin.bias.copy_(torch.from_numpy(rng.normal(0, 0.01, (N,)).astype(np.float32)))
    lin = lin.to(DEV, dtype)
    mod = q.WeightOnlyInt4Linear.from_float(lin, g)
    assert mod.weight.shape == (N // 8, K // 32, 32, 1) and mod.scales_and_zeros.shape == (K // g, N, 2)
    # quantizer parity: same closed form evaluated by torch on the CPU in the weight's dtype
    codes_cpu, scale_cpu, _ = q._quantize_int4_groupwise(lin.weight.detach().cpu(), g)
    np.testing.assert_array_equal(host(mod.weight), oracle.int4_pack_tc(codes_cpu.numpy(), 2))
    np.testing.assert_array_equal(host(mod.scales_and_zeros[..., 0]), bits_of(scale_cpu.t().contiguous()))
    x = torch.from_numpy(rng.normal(0, 1, (2, rows, K)).astype(np.float32)).to(DEV, dtype)
    y = mod(x)
    assert y.shape == (2, rows, N) and y.dtype == dtype
    xb = bits_of(x.reshape(-1, K).cpu())
    szb = bits_of(mod.scales_and_zeros.cpu())
    ref, y64 = oracle.int4_mm_tc(xb, tag, host(mod.weight), szb, g, want_f64=True)
    want = y64 + lin.bias.detach().double().cpu().numpy()[None, :]
    got = y.reshape(-1, N).float().cpu().numpy()
    assert_close_norm(got, want, 1e-2 if tag != "f32" else 1e-3, f"int4 linear {tag}")
    # the reference module test: close to the float linear
    dense = (x.reshape(-1, K).float() @ lin.weight.detach().float().t() + lin.bias.detach().float()).cpu().numpy()
    assert np.abs(got - dense).max() < 1.0


def test_act_pre_scale_is_applied():
    q = _ao()
    rng = np.random.default_rng(32)
    lin = nn.Linear(256, 64, bias=False).to(DEV, torch.float16)
    mod = q.WeightOnlyInt4Linear.from_float(lin, 64)
    x = torch.from_numpy(rng.normal(0, 1, (4, 256)).astype(np.float32)).to(DEV, torch.float16)
    pre = torch.from_numpy(rng.uniform(0.5, 2.0, (256,)).astype(np.float32)).to(DEV, torch.float16)
    plain = mod(x * pre)
    mod.act_pre_scale = pre
    assert torch.equal(mod(x), plain)


@pytest.mark.parametrize("dtype,tag", [(torch.float32, "f32"), (torch.bfloat16, "bf16"), (torch.float16, "f16")])
def test_dynamic_int8_linear_matches_oracle_chain(dtype, tag):
    q = _ao()
    rng = np.random.default_rng(33)
    M, K, N = 48, 320, 200
    x32 = rng.normal(0, 1, (3, M // 3, K)).astype(np.float32)
    w32 = rng.normal(0, 0.02, (N, K)).astype(np.float32)
    b32 = rng.normal(0, 0.01, (N,)).astype(np.float32)
    x = torch.from_numpy(x32).to(DEV, dtype)
    w = torch.from_numpy(w32).to(DEV)  # float32 master weight: cast to the activation dtype inside
    y = q.int8_dynamic_linear(x, w, torch.from_numpy(b32).to(DEV))
    assert y.shape == (3, M // 3, N) and y.dtype == torch.float32
    xq, xs = oracle.quantize_int8_rowwise(cast_bits(x32.reshape(M, K), tag), tag, 1e-5)
    wq, ws = oracle.quantize_int8_rowwise(cast_bits(w32, tag), tag, 1e-5)
    want = oracle.int8_mm_rescale(oracle.int_mm_nk(xq, wq), xs, ws) + b32[None, :]
    np.testing.assert_array_equal(host(y).reshape(M, N), want.astype(np.float32))
    # manual_int8mp_linear of the reference's test: float closed form, atol/rtol 1e-3 on small values
    ref = ((xq.astype(np.float64) * xs[:, None]) @ (wq.astype(np.float64) * ws[:, None]).T) + b32
    np.testing.assert_allclose(host(y).reshape(M, N), ref, rtol=1e-3, atol=1e-3)


def test_scaled_int8_mm_and_module():
    q = _ao()
    rng = np.random.default_rng(34)
    A = rng.integers(-127, 128, (40, 96), dtype=np.int8)
    B = rng.integers(-127, 128, (96, 24), dtype=np.int8)
    rs = rng.uniform(0.001, 0.01, 40).astype(np.float32)
    cs = rng.uniform(0.001, 0.01, 24).astype(np.float32)
    got = q.scaled_int8_mm(dev(A), dev(B), dev(rs), dev(cs))
    want = oracle.int8_mm_rescale(oracle.int_mm(A, B), rs, cs)
    np.testing.assert_array_equal(host(got), want)
    lin = nn.Linear(96, 24).to(DEV)
    mod = q.Int8DynamicLinear.from_float(lin, out_dtype=torch.bfloat16)
    x = torch.from_numpy(rng.normal(0, 1, (5, 96)).astype(np.float32)).to(DEV)
    y = mod(x)
    want = q.int8_dynamic_linear(x, lin.weight.detach(), lin.bias.detach())
    # same fp32 value rounded once to bf16 (bias inside the rounding here, outside in the reference chain)
    assert_close_norm(y.float().cpu().numpy(), want.cpu().numpy(), 1e-2, "int8 module bf16")
    model = nn.Sequential(nn.Linear(96, 64), nn.ReLU(), nn.Linear(64, 24)).to(DEV)
    dense = model(x)
    q.quantize_(model, q.Int8DynamicLinearConfig())
    assert isinstance(model[0], q.Int8DynamicLinear)
    assert_close_norm(model(x).cpu().detach().numpy(), dense.cpu().detach().numpy(), 5e-2, "int8 swapped model")


@pytest.mark.parametrize("shape", [(1, 256, 96), (7, 132, 40), (128, 512, 64)])
def test_bitnet_linear_packed(shape):
    q = _ao()
    M, K, N = shape
    rng = np.random.default_rng(612)
    w = rng.normal(0, 0.05, (N, K)).astype(np.float32)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    b = rng.normal(0, 0.1, (N,)).astype(np.float32)
    codes, scale = q.quantize_bitnet_weight(dev(w))
    ocodes, oscale = oracle.quantize_bitnet_weight(w)
    np.testing.assert_array_equal(host(codes), ocodes)
    np.testing.assert_allclose(scale.item(), oscale, rtol=1e-6)
    packed = q.pack_ternary(codes)
    y = q.bitnet_linear_packed(dev(x), packed, scale, K, bias=dev(b))
    xq, xs = oracle.quantize_int8_rowwise(x, "f32", 1e-5)
    want, _ = oracle.ternary_mm(xq, xs, oracle.pack_ternary(ocodes), float(scale.item()), K, bias=b)
    np.testing.assert_array_equal(host(y), want)
    # manual_bitnet_linear of the reference test, rtol/atol 1e-5
    ref = (xq.astype(np.int32) @ ocodes.astype(np.int32).T) * xs[:, None] * np.float32(scale.item()) + b
    np.testing.assert_allclose(host(y), ref, rtol=1e-5, atol=1e-5)
    lin = nn.Linear(K, N).to(DEV)
    mod = q.BitNetPacked2bitLinear.from_float(lin)
    assert mod(dev(x)).shape == (M, N)


def test_quantize_swaps_int4_modules():
    q = _ao()
    model = nn.Sequential(nn.Linear(256, 128, bias=False), nn.SiLU(), nn.Linear(128, 64, bias=False)).to(DEV, torch.float16)
    x = torch.randn(3, 256, device=DEV, dtype=torch.float16)
    dense = model(x)
    q.quantize_(model, q.Int4WeightOnlyConfig(groupsize=64))
    assert isinstance(model[0], q.WeightOnlyInt4Linear) and isinstance(model[2], q.WeightOnlyInt4Linear)
    y = model(x)
    assert y.shape == dense.shape
    assert (y.float() - dense.float()).abs().max().item() < 0.25 * dense.float().abs().max().item() + 0.05


# ---- int8 dynamic activation x low-bit weight linears (reference test/quantization/test_int8_dyn_act_lowbit.py) ----

def _two_layer():
    import torch.nn as nn
    return nn.Sequential(nn.Linear(64, 64, bias=False), nn.ReLU(), nn.Linear(64, 16, bias=False))


@pytest.mark.gpu
def test_8da4w_8da2w_8da1w_forward_close_to_float():
    from tensorplay_amd.ao import quantization as q
    torch.manual_seed(0)
    x = torch.randn(4, 64, device="cuda:0")
    for cfg, cls, check in ((q.int8_dynamic_activation_int4_weight(), q.Int8DynActInt4WeightLinear, "rel"),
                            (q.int8_dynamic_activation_int2_weight(), q.Int8DynActInt2WeightLinear, "rel"),
                            (q.int8_dynamic_activation_binary_weight(), q.Int8DynActBinaryWeightLinear, "cos")):
        m = _two_layer().to("cuda:0")
        ref = m(x)
        qm = q.quantize_(m, cfg)
        assert isinstance(qm[0], cls)
        out = qm(x)
        assert out.shape == (4, 16)
        if check == "rel":   # reference :30-42
            assert ((out - ref).abs().mean() / ref.abs().mean()).item() < (0.25 if cls is q.Int8DynActInt4WeightLinear else 1.0)
        else:                # reference :45-59
            assert ((out.reshape(-1) @ ref.reshape(-1)).abs() / (out.norm() * ref.norm())).item() > 0.5


@pytest.mark.gpu
def test_8da2w_matches_its_integer_formula_and_ste_gradients():
    """Forward equals (x_i8 . codes) * x_scale * w_scale bit for bit; backward is the straight-through
    estimator (reference :62-75)."""
    from tensorplay_amd import ops
    from tensorplay_amd.ao import quantization as q
    torch.manual_seed(1)
    x = torch.randn(3, 8, device="cuda:0", requires_grad=True)
    mod = q.Int8DynActInt2WeightLinear(8, 5, bias=False).to("cuda:0")
    out = mod(x)
    xq, xs = ops._quantize_int8_rowwise(x.detach(), 1e-5)
    wq, ws = ops._quantize_int2_rowwise(mod.weight.detach(), 1e-8)
    want = (xq.double() @ wq.double().T).float() * xs[:, None] * ws[None, :]
    assert torch.equal(out.detach(), want)
    out.sum().backward()
    assert mod.weight.grad.shape == (5, 8)
    torch.testing.assert_close(x.grad, torch.ones_like(out) @ mod.weight.detach(), atol=1e-4, rtol=1e-4)


@pytest.mark.gpu
def test_lowbit_quantize_kernels_match_reference_formulas():
    """reference test_int8_dyn_act_lowbit.py:95-110"""
    from tensorplay_amd import ops
    torch.manual_seed(3)
    w = torch.randn(6, 16, device="cuda:0")
    codes, scales = ops._quantize_int2_rowwise(w, 1e-8)
    scale_ref = w.abs().amax(dim=-1, keepdim=True) / 2.0
    assert bool((codes == (w / scale_ref).round().clamp(-2, 1)).all())
    assert float((scales.unsqueeze(-1) - scale_ref).abs().max()) < 1e-6
    codes_b, scales_b = ops._quantize_binary_rowwise(w, 1e-8)
    assert bool((codes_b == torch.where(w >= 0, 1, -1).to(torch.int8)).all())
    assert float((scales_b.unsqueeze(-1) - w.abs().amax(dim=-1, keepdim=True)).abs().max()) < 1e-6


# ---- on-disk format: state_dict of the packed modules ------------------------------------------------------------------

@pytest.mark.parametrize("dtype,tag", [(torch.float16, "f16"), (torch.bfloat16, "bf16")])
def test_int4_linear_loads_a_cpu_saved_state_dict(dtype, tag, tmp_path):
    """A checkpoint written by a CPU model of the reference holds `weight` in the CPU layout (uint8 [N, K/2]) and
    float32 `scales_and_zeros` (int4_weight_only.py:150-154, 180-181).  The writer here is PyTorch's own CPU pack, which
    the reference's CPU pack equals byte for byte (test_native_operator_families.py:587-589); the file goes through
    torch.save / torch.load; the loaded module must compute what the oracle computes from the same codes."""
    q = _ao()
    rng = np.random.default_rng(150)
    N, K, g, M = 272, 512, 128, 5
    codes = rng.integers(0, 16, (N, K)).astype(np.int32)
    sz32 = np.stack([rng.uniform(0.002, 0.01, (K // g, N)), rng.normal(0, 0.02, (K // g, N))], -1).astype(np.float32)
    bias = rng.normal(0, 0.01, N).astype(np.float32)
    cpu_packed = torch._convert_weight_to_int4pack_for_cpu(torch.from_numpy(codes), 2)
    assert cpu_packed.dtype == torch.uint8 and tuple(cpu_packed.shape) == (N, K // 2)
    path = tmp_path / "cpu_int4.pt"
    torch.save({"weight": cpu_packed, "scales_and_zeros": torch.from_numpy(sz32), "bias": torch.from_numpy(bias)}, path)

    mod = q.WeightOnlyInt4Linear(K, N, groupsize=g, bias=True, device=DEV, dtype=dtype)
    with pytest.warns(UserWarning, match="assuming the AVX-512 pack"):   # the tier was not stated
        result = mod.load_state_dict(torch.load(path, weights_only=True))
    assert not result.missing_keys and not result.unexpected_keys
    assert mod.weight.dtype == torch.int32 and tuple(mod.weight.shape) == (N // 8, K // 32, 32, 1)
    np.testing.assert_array_equal(host(mod.weight), oracle.int4_pack_tc(codes, 2))      # the converter, bit for bit
    szb = cast_bits(sz32, tag)
    np.testing.assert_array_equal(host(mod.scales_and_zeros), szb)                      # cast to the module dtype
    x = torch.from_numpy(rng.normal(0, 1, (M, K)).astype(np.float32)).to(DEV, dtype)
    _, y64 = oracle.int4_mm_tc(bits_of(x.cpu()), tag, oracle.int4_pack_tc(codes, 2), szb, g, round_w=False, want_f64=True)
    bias_t = torch.from_numpy(bias).to(dtype).double().numpy()
    assert_close_norm(mod(x).float().cpu().numpy(), y64 + bias_t[None, :], 2e-3 if tag == "f16" else 1e-2, "loaded int4 linear")

    # the module's own state_dict (device layout) round-trips through a file as well
    path2 = tmp_path / "device_int4.pt"
    torch.save(mod.state_dict(), path2)
    again = q.WeightOnlyInt4Linear(K, N, groupsize=g, bias=True, device=DEV, dtype=dtype)
    again.load_state_dict(torch.load(path2, weights_only=True))
    assert torch.equal(again(x), mod(x))

    # the other ISA tiers of the CPU pack, written by the library's own CPU-layout kernel
    from tensorplay_amd import ops
    for cols, split in ((32, True), (32, False)):
        other = q.WeightOnlyInt4Linear(K, N, groupsize=g, bias=True, device=DEV, dtype=dtype)
        other.cpu_pack_layout = (cols, split)
        w = ops._convert_weight_to_int4pack_for_cpu(dev(codes), 2, block_cols=cols, half_split=split).cpu()
        other.load_state_dict({"weight": w, "scales_and_zeros": torch.from_numpy(sz32), "bias": torch.from_numpy(bias)})
        assert torch.equal(other.weight, mod.weight)

    # errors: wrong extent, and a module still on the CPU
    with pytest.raises(RuntimeError, match="CPU-layout int4 weight must be"):
        mod.load_state_dict({"weight": cpu_packed[:, :-2].contiguous(), "scales_and_zeros": torch.from_numpy(sz32),
                             "bias": torch.from_numpy(bias)})
    with pytest.raises(RuntimeError, match="move the module to the GPU"):
        q.WeightOnlyInt4Linear(K, N, groupsize=g, bias=True).load_state_dict(
            {"weight": cpu_packed, "scales_and_zeros": torch.from_numpy(sz32), "bias": torch.from_numpy(bias)})


def test_bitnet_packed_linear_state_dict(tmp_path):
    """`int_data` + `scale` are the on-disk form of the packed BitNet weight (the inner tensors of the reference's
    subclass, bitnet.py:478-486): save, load into a fresh module, and the reference-style `weight` entry."""
    from types import SimpleNamespace
    q = _ao()
    rng = np.random.default_rng(611)
    M, K, N = 6, 256, 72
    w = rng.normal(0, 0.05, (N, K)).astype(np.float32)
    x = rng.normal(0, 1, (M, K)).astype(np.float32)
    lin = nn.Linear(K, N, bias=True).to(DEV)
    with torch.no_grad():
        lin.weight.copy_(dev(w))
    mod = q.BitNetPacked2bitLinear.from_float(lin)
    sd = mod.state_dict()
    assert set(sd) == {"int_data", "scale", "bias"} and sd["int_data"].dtype == torch.uint8 and sd["scale"].dim() == 0
    ocodes, oscale = oracle.quantize_bitnet_weight(w)
    np.testing.assert_array_equal(host(sd["int_data"]), oracle.pack_ternary(ocodes))
    path = tmp_path / "bitnet.pt"
    torch.save(sd, path)

    fresh = q.BitNetPacked2bitLinear(torch.zeros(N, K // 4, dtype=torch.uint8, device=DEV), 1.0, K,
                                     bias=torch.zeros(N, device=DEV))
    fresh.load_state_dict(torch.load(path, weights_only=True))
    y = fresh(dev(x))
    assert torch.equal(y, mod(dev(x)))
    xq, xs = oracle.quantize_int8_rowwise(x, "f32", 1e-5)
    want, _ = oracle.ternary_mm(xq, xs, oracle.pack_ternary(ocodes), float(sd["scale"]), K, bias=lin.bias.detach().cpu().numpy())
    np.testing.assert_array_equal(host(y), want)

    # a reference model's state_dict holds the subclass under `weight`; its inner tensors are int_data and scale
    ref_style = {"weight": SimpleNamespace(int_data=sd["int_data"].cpu(), scale=sd["scale"].cpu().reshape(1)), "bias": sd["bias"].cpu()}
    other = q.BitNetPacked2bitLinear(torch.zeros(N, K // 4, dtype=torch.uint8, device=DEV), 1.0, K, bias=torch.zeros(N, device=DEV))
    other.load_state_dict(ref_style)
    assert torch.equal(other(dev(x)), y)
    with pytest.raises(RuntimeError, match="int_data and scale"):
        other.load_state_dict({"weight": torch.zeros(3), "bias": sd["bias"]})
