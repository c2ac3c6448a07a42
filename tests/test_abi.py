"""The C-ABI library loads and exports what the headers declare (no compute calls: runs without a GPU)."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "orin_llm_amd", "liborin_fa.so")
HDR = os.path.join(ROOT, "include", "orin_fa.h")
BENCH_HDR = os.path.join(ROOT, "include", "orin_fa_bench.h")
LAYER_HDR = os.path.join(ROOT, "include", "orin_layer.h")
SHIM_HDR = os.path.join(ROOT, "include", "orin_llm_amd", "kernels.h")
REF_HDR = "/root/reference/src/kernels.h"


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def _declared_c_functions(header=HDR):
    body = _strip_comments(open(header).read())
    return sorted(set(re.findall(r"\b(orin_[a-z0-9_]+)\s*\(", body)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        pytest.fail("liborin_fa.so is not built: run `python orin_llm_amd/build.py`")
    return ctypes.CDLL(LIB)


def test_header_declares_the_expected_entry_points():
    assert _declared_c_functions() == sorted([
        "orin_fa_init", "orin_fa_set_stream", "orin_fa_workspace_bytes", "orin_fa_set_workspace",
        "orin_fa_prefill", "orin_fa_decode_ind", "orin_fa_decode_ind_static", "orin_fa_static_scratch_bytes", "orin_fa_decode_store_ind", "orin_fa_decode_rope_store_ind", "orin_fa_rope_angles_ind", "orin_fa_rope_store_batch", "orin_fa_decode_splits",
        "orin_fa_kv_store_batch", "orin_fa_kv_store_ind", "orin_fa_kv_shift", "orin_fa_rope_batch", "orin_fa_rope_ind", "orin_fa_cu_count",
        "orin_fa_device_info", "orin_fa_error_string"])


def test_measurement_aids_sit_in_their_own_header():
    assert _declared_c_functions(BENCH_HDR) == sorted([
        "orin_fa_bench_hbm_read", "orin_fa_bench_read_pattern", "orin_fa_bench_tiny_launch", "orin_fa_bench_handoff",
        "orin_fa_bench_handoff_scratch_bytes", "orin_fa_bench_handoff_stream_bytes", "orin_fa_bench_stamps"])


def test_layer_header_declares_the_expected_entry_points():
    assert _declared_c_functions(LAYER_HDR) == sorted([
        "orin_row_bytes", "orin_gemv_use_matrix_cores", "orin_gemv_row_shares", "orin_rms_norm", "orin_rms_norm_rows", "orin_quantize_activation", "orin_gemv_q8",
        "orin_gemv_q8_bias", "orin_gemv_q8_add", "orin_gemv_fused_gate_up_swiglu", "orin_gemv", "orin_dequant_row",
        "orin_swiglu", "orin_gemv_multi", "orin_gemv_multi_types", "orin_gemv_norm_gate_up_swiglu", "orin_decode_layer"])


def test_library_exports_every_declared_symbol(lib):
    for name in _declared_c_functions() + _declared_c_functions(LAYER_HDR):
        assert hasattr(lib, name), f"{name} declared in a header but not exported"


def test_the_product_library_exports_no_measurement_aid(lib):
    """The yardstick kernels and the stage-mark reader live in libraries of their own (include/orin_fa_bench.h)."""
    out = subprocess.run(["nm", "-D", "--defined-only", LIB], capture_output=True, text=True, check=True).stdout
    assert "orin_fa_bench" not in out and "_timed" not in out
    bench = os.path.join(os.path.dirname(LIB), "liborin_fa_bench.so")
    if not os.path.exists(bench):
        pytest.fail("liborin_fa_bench.so is not built: run `python orin_llm_amd/build.py`")
    aids = ctypes.CDLL(bench)
    for name in _declared_c_functions(BENCH_HDR):
        if name != "orin_fa_bench_stamps":
            assert hasattr(aids, name), f"{name} missing from liborin_fa_bench.so"
    assert not hasattr(aids, "orin_fa_prefill")


def test_timeline_build_exports_the_same_symbols():
    """liborin_fa_stamps.so is the same library with the kernels' stage marks switched on, plus the reader of their table."""
    path = os.path.join(os.path.dirname(LIB), "liborin_fa_stamps.so")
    if not os.path.exists(path):
        pytest.fail("liborin_fa_stamps.so is not built: run `python orin_llm_amd/build.py`")
    stamps = ctypes.CDLL(path)
    for name in _declared_c_functions() + _declared_c_functions(LAYER_HDR) + ["orin_fa_bench_stamps"]:
        assert hasattr(stamps, name), f"{name} missing from the timeline build"


def test_cut_off_builds_load_where_they_were_built():
    """The kernels' cut-off builds (measurement aids, results wrong by design) are built on request only
    (`python -m orin_llm_amd.build --probes`); where they exist they load and export the call they stand in for."""
    from orin_llm_amd import build as fa_build

    if not fa_build.probes_built():
        pytest.skip("cut-off builds not built (they are not part of the default build)")
    for flags in fa_build.PROBE_FLAGS:
        assert hasattr(ctypes.CDLL(fa_build.PROBE_LIB.format(flags)), "orin_fa_decode_ind")
    for flags in fa_build.PPROBE_FLAGS:
        assert hasattr(ctypes.CDLL(fa_build.PPROBE_LIB.format(flags)), "orin_fa_prefill")


def test_calls_that_need_no_device(lib):
    lib.orin_fa_workspace_bytes.restype = ctypes.c_size_t
    assert lib.orin_fa_workspace_bytes() >= 256 * 32 * (128 + 2) * 4  # 256 splits of a 32-head model
    lib.orin_fa_error_string.restype = ctypes.c_char_p
    lib.orin_fa_error_string.argtypes = [ctypes.c_int]
    assert lib.orin_fa_error_string(0) == b"ok"
    assert b"head_dim" in lib.orin_fa_error_string(-2)
    assert b"init" in lib.orin_fa_error_string(-4)
    # shape screening happens before any device work
    assert lib.orin_fa_decode_splits(12, 5, 128, 4096) == 0   # n_head % n_kv != 0
    assert lib.orin_fa_decode_splits(12, 2, 96, 4096) == 0    # head_dim
    assert lib.orin_fa_decode_splits(12, 2, 128, 32768) >= 1


def test_launch_before_init_is_refused(lib):
    """Every launch entry point checks the library state before it touches its arguments."""
    vp, ci = ctypes.c_void_p, ctypes.c_int
    if lib.orin_fa_cu_count() != 0:
        pytest.skip("the library was initialised earlier in this process")
    lib.orin_fa_prefill.argtypes = [vp] * 4 + [ci] * 6 + [ctypes.c_float]
    lib.orin_fa_decode_ind.argtypes = [vp] * 4 + [ci] * 4 + [vp, ctypes.c_float]
    assert lib.orin_fa_prefill(16, 16, 16, 16, 12, 2, 128, 4096, 0, 8, 0.1) == -4
    assert lib.orin_fa_decode_ind(16, 16, 16, 16, 12, 2, 128, 4096, 16, 0.1) == -4


def test_shim_symbols_have_the_reference_manglings():
    """The C++ shim exports llm::cuda::flash_attention / flash_attention_decode_ind / init / set_stream
    under exactly the names an engine compiled against the reference header links to."""
    out = subprocess.run(["nm", "-D", "--defined-only", LIB], capture_output=True, text=True, check=True).stdout
    syms = {line.split()[-1] for line in out.splitlines() if line.strip()}
    expected = [
        "_ZN3llm4cuda15flash_attentionEPKfPKtS4_Pfiiiiiif",
        "_ZN3llm4cuda26flash_attention_decode_indEPKfPKtS4_PfiiiiPKif",
        "_ZN3llm4cuda15rope_neox_batchEPfiiifiiPKf",
        "_ZN3llm4cuda17rope_normal_batchEPfiiifiiPKf",
        "_ZN3llm4cuda13rope_neox_indEPfiiifPKiPKf",
        "_ZN3llm4cuda15rope_normal_indEPfiiifPKiPKf",
        "_ZN3llm4cuda14kv_store_batchEPtS1_PKfS3_iiiii",
        "_ZN3llm4cuda12kv_store_indEPtS1_PKfS3_iiiPKi",
        "_ZN3llm4cuda8kv_shiftEPtS1_iiiiii",
        "_ZN3llm4cuda4initEv",
        "_ZN3llm4cuda10set_streamEPv",
        "_ZN3llm4cuda11device_infoEv",
        "_ZN3llm4cuda12scratch_sizeEii",
        "_ZN3llm4cuda14scratch_assignEPvii",
        "_ZN3llm4cuda19quantize_activationEPKfi",
        "_ZN3llm4cuda4gemvENS_5DTypeEPKvPKfPfii",
        "_ZN3llm4cuda7gemv_q8ENS_5DTypeEPKvPfii",
        "_ZN3llm4cuda12gemv_q8_biasENS_5DTypeEPKvPKfPfii",
        "_ZN3llm4cuda11gemv_q8_addENS_5DTypeEPKvPfii",
        "_ZN3llm4cuda25gemv_fused_gate_up_swigluENS_5DTypeEPKvS3_Pfii",
        "_ZN3llm4cuda11dequant_rowENS_5DTypeEPKvPfi",
        "_ZN3llm4cuda8rms_normEPKfS2_ifPf",
        "_ZN3llm4cuda13rms_norm_rowsEPKfS2_iifPf",
        "_ZN3llm4cuda6swigluEPfPKfS3_i",
    ]
    for s in expected:
        assert s in syms, s


def _decl(text, name):
    m = re.search(r"\b(?:void|int|size_t)\s+" + name + r"\s*\([^)]*\)\s*;", _strip_comments(text))
    assert m, name
    return re.sub(r"\s+", " ", m.group(0)).replace("( ", "(").strip()


@pytest.mark.skipif(not os.path.exists(REF_HDR), reason="reference tree not present on this machine")
def test_shim_header_matches_reference_declarations():
    ref, ours = open(REF_HDR).read(), open(SHIM_HDR).read()
    for name in ("flash_attention", "flash_attention_decode_ind", "kv_store_batch", "kv_store_ind", "kv_shift",
                 "rope_neox_batch", "rope_normal_batch", "rope_neox_ind", "rope_normal_ind",
                 "quantize_activation", "gemv", "gemv_q8", "gemv_q8_bias", "gemv_q8_add", "gemv_fused_gate_up_swiglu",
                 "dequant_row", "rms_norm", "rms_norm_rows", "swiglu",
                 "init", "device_info", "set_stream", "scratch_size", "scratch_assign"):
        assert _decl(ours, name) == _decl(ref, name)


def test_caller_built_against_the_reference_header_links_to_the_library(tmp_path):
    """A translation unit that includes the reference's own src/kernels.h and calls the path's
    operators the way src/model_gpu.cu does (default freq_factors included) links against
    liborin_fa.so with nothing unresolved.  Built, never run; needs the reference tree."""
    if not os.path.exists(REF_HDR):
        pytest.skip("reference tree not mounted")
    src = tmp_path / "caller.cpp"
    src.write_text('''
#include "kernels.h"
int main(int argc, char**) {
    float* q = nullptr; float* out = nullptr; uint16_t* kc = nullptr; uint16_t* vc = nullptr; int* d_pos = nullptr;
    float* k = nullptr; float* v = nullptr;
    if (argc > 1000) {  // never taken: the calls only have to resolve
        llm::cuda::init();
        llm::cuda::device_info();
        llm::cuda::set_stream(nullptr);
        void* base = nullptr;   // the engine's carve of its activation block (reference: src/model_gpu.cu:175, 208)
        if (llm::cuda::scratch_size(8960, 512) > 0) llm::cuda::scratch_assign(base, 8960, 512);
        llm::cuda::rope_neox_batch(q, 512 * 12, 128, 128, 1e6f, 0, 12);
        llm::cuda::rope_normal_batch(k, 512 * 2, 128, 128, 1e6f, 0, 2);
        llm::cuda::kv_store_batch(kc, vc, k, v, 2, 128, 4096, 0, 512);
        llm::cuda::flash_attention(q, kc, vc, out, 12, 2, 128, 4096, 0, 512, 0.088f);
        llm::cuda::rope_neox_ind(q, 12, 128, 128, 1e6f, d_pos);
        llm::cuda::rope_normal_ind(k, 2, 128, 128, 1e6f, d_pos);
        llm::cuda::kv_store_ind(kc, vc, k, v, 2, 128, 4096, d_pos);
        llm::cuda::flash_attention_decode_ind(q, kc, vc, out, 12, 2, 128, 4096, d_pos, 0.088f);
        llm::cuda::kv_shift(kc, vc, 28, 2, 128, 4096, 4, 2046);
        // the rest of the decode layer (reference: src/model_gpu.cu:251-293, 303-306)
        const void* W = nullptr; float* x = nullptr; float* y = nullptr; const float* w = nullptr;
        llm::cuda::dequant_row(llm::DType::Q4_K, W, x, 1536);
        llm::cuda::rms_norm(x, w, 1536, 1e-6f, y);
        llm::cuda::quantize_activation(y, 1536);
        llm::cuda::gemv_q8(llm::DType::Q4_K, W, q, 1536, 1536);
        llm::cuda::gemv_q8_bias(llm::DType::Q6_K, W, w, v, 1536, 256);
        llm::cuda::rms_norm_rows(q, w, 12, 128, 1e-6f, q);
        llm::cuda::gemv_q8_add(llm::DType::Q4_K, W, x, 1536, 1536);
        llm::cuda::gemv_fused_gate_up_swiglu(llm::DType::Q4_K, W, W, y, 1536, 8960);
        llm::cuda::swiglu(y, y, y, 8960);
        llm::cuda::gemv(llm::DType::Q6_K, W, x, y, 1536, 151936);
    }
    return 0;
}
''')
    exe = tmp_path / "caller"
    r = subprocess.run(["g++", "-std=c++17", "-I", os.path.dirname(REF_HDR), "-I", "/root/reference/include", str(src),
                        "-o", str(exe), "-L", os.path.dirname(LIB), "-lorin_fa", "-Wl,--no-undefined",
                        "-Wl,--allow-shlib-undefined", "-Wl,-rpath," + os.path.dirname(LIB)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
