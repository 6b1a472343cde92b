"""CPU: the C-ABI library loads and exports every symbol the headers declare (no compute calls)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "turbo-lossless_amd", "libturbo12.so")


def declared_functions(path):
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    text = re.sub(r"^\s*#[^\n]*", "", text, flags=re.M)
    text = re.sub(r"typedef\s+struct\s+\w+\s*\{.*?\}\s*\w+\s*;", "", text, flags=re.S)
    return set(re.findall(r"\b(\w+)\s*\([^;{]*\)\s*;", text))


def test_library_exports_declared_c_abi():
    assert os.path.exists(LIB), "build first: python turbo-lossless_amd/build.py"
    lib = ctypes.CDLL(LIB)
    names = declared_functions(os.path.join(ROOT, "include", "t12_abi.h"))
    assert {"t12_gemv", "t12_gemm", "t12_decompress", "launch_split12_v2_async", "launch_split12_batch8_async",
            "t12_pack_planes"} <= names
    missing = [n for n in sorted(names) if not hasattr(lib, n)]
    assert not missing, missing


def test_library_exports_every_declaration_of_every_header():
    lib = ctypes.CDLL(LIB)
    for header in ("t12_abi.h", "t12_glue.h", "t12_engine.h"):
        names = declared_functions(os.path.join(ROOT, "include", header))
        assert len(names) >= 15, (header, names)
        missing = [n for n in sorted(names) if not hasattr(lib, n)]
        assert not missing, (header, missing)


def test_every_exported_c_symbol_is_declared_in_a_header():
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", LIB], capture_output=True, text=True).stdout
    exported = {ln.split()[2] for ln in out.splitlines() if len(ln.split()) == 3 and ln.split()[1] == "T"
                and not ln.split()[2].startswith("_")}
    declared = set()
    for header in ("t12_abi.h", "t12_glue.h", "t12_engine.h"):
        declared |= declared_functions(os.path.join(ROOT, "include", header))
    assert not sorted(exported - declared), sorted(exported - declared)


def test_library_exports_glue_and_engine_c_face():
    lib = ctypes.CDLL(LIB)
    glue = ["launch_embed_lookup", "launch_rms_norm_bf16_batch", "launch_add_rms_norm_bf16_batch",
            "launch_silu_mul_bf16_batch", "launch_add_batch", "launch_rope_batch", "launch_store_kv_batch",
            "launch_attention_all_heads", "launch_attention_all_heads_batch", "launch_flash_attention",
            "launch_flash_attention_batch", "launch_rope_store_kv", "launch_rope_init", "launch_argmax",
            "launch_argmax_batch"]                      # engine/inference.cpp:9-20, sampler.cpp:4-5
    other_build = ["nv_launch_split12_v2_async", "nv_launch_split12_v2_dual_async", "nv_launch_patches_async",
                   "nv_launch_patches_batch_async", "nv_launch_split12_fused_gemm_async",
                   "nv_launch_split12_cublas_batch_async"]                         # engine/inference.cpp:33-41
    glue = glue + other_build
    engine = ["t12_engine_load", "t12_engine_create_state", "t12_engine_forward", "t12_engine_generate",
              "t12_engine_sample", "t12_engine_free_state", "t12_engine_free_model"]
    missing = [n for n in glue + engine if not hasattr(lib, n)]
    assert not missing, missing


def test_cpp_api_symbols_present():
    """The C++ API of include/turbo/*.h is exported with C++ linkage (mangled names contain the identifiers)."""
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", LIB], capture_output=True, text=True).stdout
    for ident in ["load_model", "free_model", "create_inference_state", "free_inference_state", "forward",
                  "generate", "init_sampler", "sample_greedy", "sample_greedy_batch", "create_synthetic_model",
                  "save_model", "prefill", "shift_context", "chat_turn",
                  "load_tokenizer", "free_tokenizer", "tokenize", "detokenize", "detokenize_one"]:   # engine/tokenizer.h:19-23
        assert re.search(r"_Z\d+%s" % ident, out), ident


def test_error_paths_without_gpu():
    lib = ctypes.CDLL(LIB)
    lib.t12_last_error.restype = ctypes.c_char_p
    lib.t12_version.restype = ctypes.c_char_p
    assert lib.t12_version().startswith(b"turbo12")
    assert lib.t12_gemv(None, 0, None, 0, None) == -1          # rejected on the host, nothing launched
    assert b"nseg" in lib.t12_last_error()
    assert lib.t12_gemm(None, 1, None, 0, 0, 0, 0, None) == -1
    assert lib.t12_decompress(None, None, 0, None, None, None, None, 4, 4, 0, None) == -1
    hist = (ctypes.c_uint64 * 256)()
    lib.t12_pack_base_exp.argtypes = [ctypes.POINTER(ctypes.c_uint64)]
    assert lib.t12_pack_base_exp(hist) == -1                    # empty histogram -> -1 (split12_pack.c:36)
    hist[120] = 5; hist[140] = 5
    assert lib.t12_pack_base_exp(hist) == 105                   # earliest best window [106,120] -> base 105
