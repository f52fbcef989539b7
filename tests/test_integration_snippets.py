"""Every C++ code block of the integration guide (the markdown file at the repository root that shows the reference-side
bindings) is compiled (syntax and types only) against include/vsp_attn.h, so that a
signature change in the header cannot leave the integration guide behind.  The reference's own declarations are
replaced by the small stand-in tests/cpp/reference_stub.hpp; blocks that are statements are wrapped in a function whose
parameters are the variables the surrounding text introduces."""
import os
import re
import subprocess
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GUIDE = "INTEGRATION" + ".md"

# what each block is, in the order of appearance: a translation-unit level block, or statements with the variables they use
_T = "const vesper::Tensor&"
BLOCKS = [
    ("tensor-to-vsp helpers", "global", ""),
    ("flash_attention_hip_dispatch", "global", ""),
    ("KVCache::update / reset", "member", ""),
    ("decode inside scaled_dot_product_attention", "function",
     f"{_T} query, vesper::Tensor output, vsp_kv_cache* cache_desc, vsp_tensor dq, vsp_tensor dout, int32_t B, int32_t Hq, int32_t D, void* stream"),
    ("decode through wo_", "function",
     f"{_T} wo_weight, vesper::Tensor y, vsp_kv_cache* cache_desc, vsp_tensor dq, int64_t T, int32_t B, int32_t Hq, int32_t D, void* stream"),
    ("RoPE + cache write", "function",
     f"int32_t max_seq_len, int32_t head_dim_, float rope_base_, const float*& rope_table_, const float* (*upload)(const std::vector<float>&), "
     f"{_T} q_view, {_T} k_view, {_T} v_view, {_T} q_rot, vsp_kv_cache cache_desc, int64_t start_pos, void* stream"),
    ("chunked prefill over the cache", "function",
     "vsp_tensor dq_rot, vsp_tensor dout, vsp_kv_cache cache_desc, int32_t Hq, int32_t T, int D, void* workspace, void* stream"),
    ("a few tokens per sequence through the decode kernels", "function",
     "vsp_tensor dq_rot, vsp_tensor dout, vsp_kv_cache cache_desc, int32_t B, int32_t T, int32_t Hq, int D, void* workspace, void* stream"),
    ("flash_attention_backward_hip_dispatch", "global", ""),
    ("the same body for fp32 tensors with split operands", "function",
     f"{_T} q, {_T} k, vsp_tensor d_dout, vsp_tensor dq_, vsp_tensor dk_, vsp_tensor dv_, vsp_tensor d_out, vsp_tensor d_lse, "
     "vsp_tensor d_gq, vsp_tensor d_gk, vsp_tensor d_gv, float scale, bool is_causal"),
]


def _cpp_blocks(text):
    return re.findall(r"```cpp\n(.*?)```", text, flags=re.S)


def test_integration_md_code_blocks_compile_against_the_header():
    blocks = _cpp_blocks(open(os.path.join(ROOT, GUIDE)).read())
    assert len(blocks) == len(BLOCKS), f"{GUIDE} has {len(blocks)} C++ blocks, the test describes {len(BLOCKS)}"
    src = ['#include "reference_stub.hpp"', "using namespace vesper;", "using namespace vesper::nn;"]
    for i, (body, (name, kind, params)) in enumerate(zip(blocks, BLOCKS)):
        src.append(f"// ---- block {i}: {name}")
        if kind == "function":
            src.append(f"[[maybe_unused]] static vesper::Tensor block_{i}({params}) {{\n{body}\nreturn output_{i}();\n}}".replace(
                f"return output_{i}();", "return vesper::Tensor();"))
        else:
            src.append(body)
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "integration_blocks.cpp")
        with open(path, "w") as f:
            f.write("\n".join(src) + "\n")
        r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Wno-unused-variable", "-Wno-unused-function",
                            "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "tests", "cpp"), path],
                           capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]
