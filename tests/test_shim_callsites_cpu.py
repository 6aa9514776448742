"""CPU: the reference's own `at::cuda::launch_*` call expressions compile against include/ptm_at_cuda_shim.h.

The call expressions are cut out of the reference checkout at test time (torch/io/gguf_model.h: forward_decode, KVCache::append,
gemv_scratch, fused_gate_up_gemv, matmul_q, the prefill layer, generate's argmax), each one verbatim, and wrapped in a
function whose parameters are stand-ins for the variables it names (tensors with data_ptr<float>(), weight handles with
gpu_data / rows / cols / row_stride_bytes, plain ints, floats and pointers).  g++ -fsyntax-only then checks every name, the
argument count and every argument type against the shim.  Nothing of the reference is stored here; without the checkout the
test is skipped."""
import os
import re
import shutil
import subprocess

import pytest

from conftest import ROOT

REF = "/root/reference/torch/io/gguf_model.h"
# line windows of gguf_model.h that hold at::cuda:: calls (wide on purpose: the extraction keys on the call syntax)
WINDOWS = [(360, 390), (505, 540), (600, 620), (1320, 1345), (1425, 1445), (2610, 2630), (2660, 3095), (3112, 3170),
           (4845, 4860), (6915, 6975), (7000, 7030), (7190, 7215), (7390, 7415), (7460, 7480), (7520, 7535), (7620, 7640)]

INT = "long"
SCALARS = {
    **{n: INT for n in ("H K K_lm K_out M1 M2 N N_gate N_lm N_out N_up Ni Nr V cols head_dim inter kv_dim max_K max_seq "
                        "n_heads n_kv_heads num_new past_len position_offset q_dim rows row_stride_bytes seq_len total_seq "
                        "cur next i layer_idx").split()},
    **{n: "float" for n in "eps scale freq_base".split()},
    "add_one": "bool",
    **{n: "float*" for n in "x_ptr y_ptr y y_gate y_up".split()},
    **{n: "const float*" for n in "normed_ptr logit_row".split()},
    "d_argmax_idx": "int64_t*", "d_past_len_": "int64_t*", "d_token_id_": "int*", "lm_head_fp16_": "void*",
    "gpu_data": "void*", "fp16_data": "void*",
    "s": "cudaStream_t", "stream": "cudaStream_t",
}
TENSORS = "a b gate up hidden k v q new_k new_v output result weight float_w emb_gpu_ output_norm output_weight".split()
HANDLES = "qw qg qu q_output_weight".split()

PRELUDE = r"""
#include "ptm_at_cuda_shim.h"
#include <vector>
struct MockTensor {
    template <typename T> T* data_ptr() const { return nullptr; }
    template <typename T> T* mutable_data_ptr() const { return nullptr; }
    bool defined() const { return true; }
    long numel() const { return 0; }
    long size(int) const { return 0; }
    operator const float*() const { return nullptr; }   // a name that is a tensor at one call site and a pointer at another
};
struct MockQW { void* gpu_data; void* fp16_data; long rows, cols, row_stride_bytes; };
struct MockConfig { float rms_norm_eps, rope_freq_base; bool gemma_norm_add_one; long vocab_size; };
"""


def extract_calls():
    lines = open(REF, encoding="utf-8", errors="replace").read().split("\n")
    calls = []
    for a, b in WINDOWS:
        text = "\n".join(lines[a - 1:b])
        for m in re.finditer(r"at::cuda::(launch_\w+|flash_decode_num_splits|init_cuda_kernel_smem_attributes)\s*\(", text):
            i, depth = m.end(), 1
            while depth:
                depth += {"(": 1, ")": -1}.get(text[i], 0)
                i += 1
            calls.append((a + text[:m.start()].count("\n"), text[m.start():i]))
    return calls


def members(calls, root):
    """struct body for `root` (layer / sp / kv_cache) from the member accesses the calls make"""
    out = {}
    for _, c in calls:
        for name, idx, rest in re.findall(root + r"\.(\w+)(\[\w+\])?(\.\w+)?", c):
            if rest in (".data_ptr", ".mutable_data_ptr", ".defined"):
                t = "MockTensor"
            elif rest:
                t = "MockQW"
            elif name == "max_seq":
                t = "long"
            else:
                t = "void*" if "fp16" in name else "float*"
            out[name] = f"std::vector<{t}> {name};" if idx else f"{t} {name};"
    return "\n    ".join(out[k] for k in sorted(out))


def params_of(call):
    body = re.sub(r"at::cuda::\w+", "", call)
    body = re.sub(r"static_cast<\w+>", "", body)
    body = re.sub(r"(data_ptr|mutable_data_ptr)<float>", "", body)
    roots = []
    for m in re.finditer(r"(?<![\w\.>:])([A-Za-z_]\w*)", body):
        n = m.group(1)
        if n in ("nullptr", "true", "false", "int", "float", "std", "sqrt") or n in roots:
            continue
        roots.append(n)
    ps = []
    for n in roots:
        if n == "layer": ps.append("MockLayer& layer")
        elif n == "sp": ps.append("MockScratch& sp")
        elif n == "kv_cache": ps.append("MockKV& kv_cache")
        elif n == "config": ps.append("MockConfig& config")
        elif n in ("key_cache", "value_cache"): ps.append(f"std::vector<MockTensor>& {n}")
        elif n in ("key_cache_fp16", "value_cache_fp16"): ps.append(f"std::vector<void*>& {n}")
        elif n == "x": ps.append("MockTensor& x")      # float* in gemv_scratch, a tensor in apply_rope
        elif n in TENSORS:  # `hidden` is a tensor in one function of the reference and a row width in another
            ps.append(f"MockTensor& {n}" if re.search(rf"\b{n}\.", call) else f"{INT} {n}")
        elif n in HANDLES: ps.append(f"MockQW& {n}")
        elif n in SCALARS: ps.append(f"{SCALARS[n]} {n}")
        else: raise AssertionError(f"no stand-in type for `{n}` in: {call}")
    return ", ".join(ps)


@pytest.mark.skipif(not os.path.exists(REF), reason="reference checkout not present")
def test_reference_call_sites_compile_against_the_shim(tmp_path):
    if not (shutil.which("g++") and os.path.isdir("/opt/rocm/include")):
        pytest.skip("no g++ / ROCm headers")
    calls = extract_calls()
    names = {re.match(r"at::cuda::(\w+)", c).group(1) for _, c in calls}
    # every launcher forward_decode / forward / KVCache / gemv_scratch / matmul_q name must be among them
    for must in ("launch_fused_qknorm_rope_kvwrite", "launch_fused_qknorm_rope_kvwrite_graph", "launch_flash_decode",
                 "launch_flash_decode_fp16", "launch_flash_decode_graph", "launch_mul_scalar", "launch_kv_cache_write",
                 "launch_fp16_kv_cache_write", "launch_rope", "launch_causal_attention", "launch_concat",
                 "launch_inference_gemv", "launch_gemv", "launch_cublas_hgemv", "launch_fp16_gemv",
                 "launch_q4km_persistent_gemv", "launch_q4km_persistent_gemv_accumulate", "launch_q6k_gemv",
                 "launch_q5k_gemv", "launch_q4km_fused_rmsnorm_qkv_gemv", "launch_q4km_fused_rmsnorm_gate_up_gemv",
                 "launch_q4km_fused_gate_up_gemv", "launch_rms_norm", "launch_per_head_rms_norm", "launch_silu_mul",
                 "launch_add", "launch_copy", "launch_embedding_lookup", "launch_argmax", "launch_dequant_q4k_to_fp16",
                 "flash_decode_num_splits", "init_cuda_kernel_smem_attributes"):
        assert must in names, f"{must}: call site not found in the reference windows"
    assert len(calls) >= 60
    src = [PRELUDE,
           "struct MockLayer {\n    " + members(calls, "layer") + "\n};",
           "struct MockScratch {\n    " + members(calls, "sp") + "\n};",
           "struct MockKV {\n    " + members(calls, "kv_cache") + "\n};"]
    for k, (line, call) in enumerate(calls):
        src.append(f"// gguf_model.h:{line}\nvoid call_{k}({params_of(call)}) {{\n    {call};\n}}")
    f = tmp_path / "callsites.cpp"
    f.write_text("\n".join(src))
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Werror", "-Wno-unused-parameter",
                        "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include"), str(f)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-4000:]


def test_shim_context_setter_and_integration_snippet_compile(tmp_path):
    """How a maintainer of the reference sets the shim's context: from the model's own fields, inside a member function, in front
    of the launcher calls.  That snippet compiles."""
    if not (shutil.which("g++") and os.path.isdir("/opt/rocm/include")):
        pytest.skip("no g++ / ROCm headers")
    f = tmp_path / "ctx.cpp"
    f.write_text(r"""
#include "ptm_at_cuda_shim.h"
struct KV { long max_seq; float* k; float* v; };
struct Config { bool rope_neox; float rope_freq_base; };
struct Model {
    KV kv_cache; Config config; const float* rope_table_gpu_ = nullptr; int64_t* d_past_len_ = nullptr;
    void forward_decode(float* q, float* k, const float* v, cudaStream_t s) {
        at::cuda::ptm_shim_set_context(static_cast<int>(kv_cache.max_seq), config.rope_neox ? 1 : 0, rope_table_gpu_);
        at::cuda::launch_fused_qknorm_rope_kvwrite_graph(q, k, v, nullptr, nullptr, kv_cache.k, kv_cache.v, 32, 8, 128,
                                                         d_past_len_, config.rope_freq_base, 1e-6f, false, s);
        at::cuda::launch_fused_qknorm_rope_kvwrite(q, k, v, nullptr, nullptr, kv_cache.k, kv_cache.v, 32, 8, 128, 7,
                                                   config.rope_freq_base, 1e-6f, false, 7, s);
    }
};
int main() { return at::cuda::ptm_shim_context().max_seq == 4096 ? 0 : 1; }
""")
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__",
                        "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include"), str(f)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    shim = open(os.path.join(ROOT, "include", "ptm_at_cuda_shim.h")).read()
    body = re.sub(r"/\*.*?\*/", "", shim, flags=re.S)
    assert "launch_quantize_q8_1" not in body and "launch_q4km_q8_gemv" not in body   # 36-byte block contract not offered
    assert "PTM_SHIM_MAX_SEQ" not in shim and "PTM_SHIM_ROPE_NEOX" not in shim
