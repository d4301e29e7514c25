"""The float32 path is true float32 by construction: the float32 code of every kernel file lies in regions in
which reduced-precision matrix instructions and hardware approximations cannot be named (csrc/exact_begin.h),
and the float32 builds of the matrix products cannot name a bfloat16 type at all.  computerex/dlgo keeps
activations, cache and accumulators in float32 (models/llm/forward.go:13-28, memory/kvcache.go:5-9).

These tests fail if a kernel is moved out of its region, if a region stops refusing a name, or if the compiler
flags gain a fast-math switch."""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

from dlgo_amd.kernels import build

CSRC = build.CSRC

# kernels that may use bfloat16 MFMA and the hardware's exp2: they only ever run on bfloat16 operands
BF16_ONLY = {"attn_prefill_kernel", "attn_decode_kernel", "attn_decode_lds_kernel"}


def _regions(path):
    """For each line of the file: inside an exact region or not."""
    inside, flags = False, []
    for line in open(path).read().split("\n"):
        if re.match(r'\s*#include "exact_begin.h"', line):
            assert not inside, f"{path}: nested exact region"
            inside = True
        flags.append(inside)
        if re.match(r'\s*#include "exact_end.h"', line):
            assert inside, f"{path}: exact_end.h without a begin"
            inside = False
    return flags


def _kernels(path):
    """(name, first line, last line) of every __global__ function of the file."""
    lines = open(path).read().split("\n")
    out = []
    for i, line in enumerate(lines):
        if "__global__" not in line or line.lstrip().startswith("//"):
            continue
        head = " ".join(lines[i:i + 4])
        m = re.search(r"\bvoid\s+(\w+)\s*\(", head)
        assert m, f"{path}:{i + 1}: cannot read the kernel's name"
        depth, j, seen = 0, i, False
        while True:
            depth += lines[j].count("{") - lines[j].count("}")
            seen = seen or "{" in lines[j]
            if seen and depth == 0:
                break
            j += 1
        out.append((m.group(1), i, j))
    return out


def test_every_float32_kernel_lies_in_an_exact_region():
    found_bf16_only = set()
    for name in sorted(os.listdir(CSRC)):
        if not name.endswith(".hip"):
            continue
        path = os.path.join(CSRC, name)
        text = open(path).read()
        if '#include "gemm_common.h"' in text:
            continue            # guarded as a whole per element type, see the next test
        flags = _regions(path)
        kernels = _kernels(path)
        assert kernels, f"{name}: no kernels found"
        for kernel, a, b in kernels:
            if kernel in BF16_ONLY:
                found_bf16_only.add(kernel)
                assert not any(flags[a:b + 1]), f"{name}: {kernel} is listed as bfloat16-only but lies in an exact region"
                continue
            assert all(flags[a:b + 1]), f"{name}: kernel {kernel} (lines {a + 1}-{b + 1}) is not inside an exact region"
    assert found_bf16_only == BF16_ONLY
    # the float32 kernels and the merge of the float32 partial results are where they are believed to be
    att = os.path.join(CSRC, "attention.hip")
    names = {k for k, _, _ in _kernels(att)}
    assert {"attn_rows_kernel", "attn_prefill_f32_kernel", "attn_decode_f32_kernel", "attn_combine_kernel"} <= names
    flags = _regions(att)
    for i, line in enumerate(open(att).read().split("\n")):
        if "merge_weight<true>(float x)" in line:
            assert flags[i] and "expf(x)" in line
        if "merge_weight<false>(float x)" in line:
            assert not flags[i]


def test_matrix_products_open_the_region_for_the_float32_build():
    text = open(os.path.join(CSRC, "gemm_common.h")).read()
    m = re.search(r'#if DLGO_ELEM == DLGO_DTYPE_F32\s*\n#define DLGO_EXACT_NO_BF16 1\s*\n#include "exact_begin.h"\s*\n#endif', text)
    assert m, "gemm_common.h no longer opens an exact region for the float32 build"
    before = text[:m.start()]
    assert "__device__" not in before and "__global__" not in before, "code stands before the float32 build's exact region"
    for name in ("gemm.hip", "gemm_rows.hip"):
        src = open(os.path.join(CSRC, name)).read()
        first_include = re.search(r'^#include "(\w+\.h)"', src, re.M).group(1)
        assert first_include == "gemm_common.h"
        # bfloat16 specialisations exist only in the bfloat16 build
        for m2 in re.finditer(r"^template <> struct \w+<bf16_t>", src, re.M):
            upto = src[:m2.start()]
            assert upto.count("#if DLGO_ELEM == DLGO_DTYPE_BF16") > upto.count("#endif") - upto.count("#if DLGO_ELEM == DLGO_DTYPE_F32"), \
                f"{name}: a bfloat16 specialisation outside #if DLGO_ELEM == DLGO_DTYPE_BF16"


def test_no_fast_math_flag():
    joined = " ".join(build.FLAGS)
    for bad in ("fast-math", "unsafe", "ffp-contract=fast ", "finite-math", "fno-honor", "approx", "freciprocal", "cuda-approx",
                "fgpu-approx", "no-correctly-rounded", "denormals"):
        assert bad not in joined, f"compiler flag {bad!r} would weaken float32 arithmetic"


_PROBES = {
    "exp2": "__builtin_amdgcn_exp2f(x)",
    "rcp": "__builtin_amdgcn_rcpf(x)",
    "rsq": "__builtin_amdgcn_rsqf(x)",
    "expf_fast": "__expf(x)",
    "fdividef": "__fdividef(x, 3.0f)",
    "helper": "fast_exp2(x)",
    "bf16_mfma": "__builtin_amdgcn_mfma_f32_16x16x32_bf16(a, a, c, 0, 0, 0)[0]",
    "bf16_mfma_32": "__builtin_amdgcn_mfma_f32_32x32x16_bf16(a, a, d, 0, 0, 0)[0]",
    "xf32_mfma": "__builtin_amdgcn_mfma_f32_16x16x8_xf32(v2, v2, c, 0, 0, 0)[0]",
}


def _syntax_check(source, defines=()):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc is not installed here")
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "probe.hip")
        with open(path, "w") as f:
            f.write(source)
        r = subprocess.run([hipcc, f"--offload-arch={build.ARCH}", "-fsyntax-only", "-std=c++17", "-I", CSRC, *defines, path],
                           capture_output=True, text=True, env=dict(os.environ, HOME=d))
    return r.returncode, r.stdout + r.stderr


_PRELUDE = """#include "common.h"
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
__device__ float fast_exp2(float x) { return x; }
"""
_BODY = """__device__ float probe(float x, bf16x8_t a, f32x4_t c, f32x16_t d, f32x2_t v2) { return %s; }
"""


def test_an_exact_region_refuses_every_approximation_by_name():
    # outside a region all of them compile: the probes are valid code
    rc, log = _syntax_check(_PRELUDE + "".join(_BODY.replace("probe", f"probe_{k}") % v for k, v in _PROBES.items()))
    assert rc == 0, log
    # inside, each is an error that names the guard; after the region they compile again
    for key, expr in _PROBES.items():
        src = _PRELUDE + '#include "exact_begin.h"\n__device__ float fine(float x) { return expf(x) / (1.0f + sqrtf(x)); }\n' + _BODY % expr + '#include "exact_end.h"\n'
        rc, log = _syntax_check(src)
        assert rc != 0 and "DLGO_NOT_IN_FLOAT32_CODE" in log, f"{key}: an exact region let {expr} through\n{log}"
    src = _PRELUDE + '#include "exact_begin.h"\n#include "exact_end.h"\n' + _BODY % _PROBES["exp2"]
    rc, log = _syntax_check(src)
    assert rc == 0, log


def test_the_float32_products_cannot_name_bfloat16():
    tail = "__device__ float probe(float x) { return %s; }\n"
    for expr in ("(float)(__bf16)x", "bf16_to_f32((bf16_t)1)", "(float)f32_to_bf16(x)", "__builtin_amdgcn_rcpf(x)"):
        rc, log = _syntax_check('#include "gemm_common.h"\n' + tail % expr, ["-DDLGO_ELEM=0"])
        assert rc != 0 and "DLGO_NOT_IN_FLOAT32_CODE" in log, f"the float32 build of the products let {expr} through\n{log}"
        rc, log = _syntax_check('#include "gemm_common.h"\n' + tail % expr, ["-DDLGO_ELEM=1"])
        assert rc == 0, log
    # and the real files pass with the guard on
    for name in ("gemm.hip", "gemm_rows.hip"):
        rc, log = _syntax_check(f'#include "{name}"\n', ["-DDLGO_ELEM=0"])
        assert rc == 0, log
