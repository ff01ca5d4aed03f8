"""Text-level checks of integration/tpq_gfx950_registrar.cpp, the C++ file that registers the library's kernels in a
TensorPlay build.  It cannot be compiled here (the reference's Tensor.h includes a header its code generator writes
at build time), so what can be checked without a compiler is:

* every tpq_* function it calls is declared in include/tpq.h with the same number of arguments;
* with the reference checkout present (this container only): every registered op name is an operator of
  config/native_functions.yaml, is registered by the reference on the CUDA key under the same bare name, and the
  function registered here has the same return type and parameter types as the kernel it replaces.
"""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REGISTRAR = os.path.join(ROOT, "integration", "tpq_gfx950_registrar.cpp")
REFERENCE = "/root/reference"

EXPECTED_OPS = {"_quantize_int8_rowwise", "_quantize_int4_rowwise", "_quantize_int2_rowwise", "_quantize_binary_rowwise",
                "_int8_mm_rescale", "_int_mm", "_int_mm.out", "_convert_weight_to_int4pack", "_weight_int4pack_mm",
                "_weight_int8pack_mm", "quantize_affine", "dequantize_affine"}


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _split_top_level(args):
    out, depth, cur = [], 0, ""
    for ch in args:
        if ch in "(<[{":
            depth += 1
        elif ch in ")>]}":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur.strip())
    return out


def _balanced(text, open_at):
    """text[open_at] == '(' -> the text between it and its matching ')'."""
    depth = 0
    for i in range(open_at, len(text)):
        if text[i] == "(":
            depth += 1
        elif text[i] == ")":
            depth -= 1
            if depth == 0:
                return text[open_at + 1:i]
    raise AssertionError("unbalanced parentheses")


def _registrations(text):
    return dict(re.findall(r'm\.impl\("([^"]+)",\s*([A-Za-z0-9_]+)\)', text))


def _param_type(param):
    """'const Tensor& self' -> 'const Tensor&'; 'int64_t q_group_size' -> 'int64_t' (default values dropped)."""
    param = param.split("=")[0].strip()
    m = re.match(r"(.*?[\s&*>])([A-Za-z_][A-Za-z0-9_]*)$", param)
    return re.sub(r"\s+", " ", (m.group(1) if m else param).strip()).replace(" &", "&").replace("tensorplay::", "")


def _signature(text, name):
    """(return type, [parameter types]) of the definition of `name` in C++ source text."""
    for m in re.finditer(r"([A-Za-z_:<>,\s&]+?)\b" + re.escape(name) + r"\s*\(", text):
        params = _balanced(text, m.end() - 1)
        after = text[m.end() + len(params):].lstrip(") \n\t")
        if not after.startswith("{"):
            continue  # a call or a declaration, not the definition
        ret = re.sub(r"\s+", " ", m.group(1).strip().split("\n")[-1].strip()).replace(" &", "&")
        ret = re.sub(r"^(static|inline)\s+", "", ret)
        return ret, [_param_type(p) for p in _split_top_level(params)]
    raise AssertionError(f"no definition of {name} found")


def test_registrar_registers_the_twelve_ops_under_bare_names():
    regs = _registrations(_strip_comments(open(REGISTRAR).read()))
    assert set(regs) == EXPECTED_OPS
    assert all("::" not in name for name in regs), "contract ops are keyed by bare name"
    assert "TENSORPLAY_LIBRARY_IMPL(CUDA," in open(REGISTRAR).read()


def test_every_library_call_matches_the_header():
    header = _strip_comments(open(os.path.join(ROOT, "include", "tpq.h")).read())
    declared = {}
    for m in re.finditer(r"\b(tpq_[a-z0-9_]+)\s*\(", header):
        declared[m.group(1)] = len(_split_top_level(_balanced(header, m.end() - 1)))
    text = _strip_comments(open(REGISTRAR).read())
    calls = [(m.group(1), m.end() - 1) for m in re.finditer(r"\b(tpq_[a-z0-9_]+)\s*\(", text)]
    assert len(calls) >= 10
    for name, at in calls:
        assert name in declared, f"{name} is not declared in include/tpq.h"
        args = _split_top_level(_balanced(text, at))
        want = declared[name] if _balanced(header, header.index(name + "(") + len(name)).strip() != "void" else 0
        assert len(args) == want, f"{name}: {len(args)} arguments passed, {want} declared"


@pytest.mark.skipif(not os.path.isdir(REFERENCE), reason="the reference checkout is only present in the build container")
def test_signatures_equal_the_kernels_they_replace():
    regs = _registrations(_strip_comments(open(REGISTRAR).read()))
    ours = _strip_comments(open(REGISTRAR).read())
    yaml = open(os.path.join(REFERENCE, "config", "native_functions.yaml")).read()
    cuda_dir = os.path.join(REFERENCE, "p10", "src", "backend", "cuda")
    sources = {f: _strip_comments(open(os.path.join(cuda_dir, f)).read())
               for f in ("QuantGemmKernels.cu", "IntMM.cu", "LowBitGemmKernels.cu", "AffineQuantKernels.cu")}
    for op, fn in regs.items():
        assert re.search(r"^- func: " + re.escape(op) + r"\(", yaml, flags=re.M), f"{op} is not in native_functions.yaml"
        theirs = None
        for fname, text in sources.items():
            block = re.search(r"TENSORPLAY_LIBRARY_IMPL\(CUDA,[^)]*\)\s*\{(.*?)\n\}", text, flags=re.S)
            ref_regs = _registrations(block.group(1)) if block else {}
            if op in ref_regs:
                theirs = _signature(text, ref_regs[op])
        assert theirs is not None, f"the reference registers no CUDA kernel named {op}"
        mine = _signature(ours, fn)
        assert mine == theirs, f"{op}: {mine} here, {theirs} in the reference"
