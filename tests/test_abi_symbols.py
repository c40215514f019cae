"""CPU-side checks of the drop-in boundary: the built libraries load and export every symbol
the headers under include/ declare (no compute is called here)."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "xfastertransformer_amd")
LIB_HIP = os.path.join(PKG, "libxft_hip.so")
LIB_LAYERS = os.path.join(PKG, "libxft_layers.so")


def _declared_c_symbols():
    text = open(os.path.join(ROOT, "include", "xft_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xfthip_[a-z0-9_]+)\s*\(", text)))


def _exported(path):
    out = subprocess.check_output(["nm", "-D", "--defined-only", path], text=True)
    return {line.split()[-1] for line in out.splitlines() if line.strip()}


@pytest.mark.skipif(not os.path.exists(LIB_HIP), reason="library not built (run __graft_entry__.build())")
def test_c_abi_exports_every_declared_symbol():
    declared = _declared_c_symbols()
    assert len(declared) > 40
    exported = _exported(LIB_HIP)
    missing = [s for s in declared if s not in exported]
    assert not missing, missing
    lib = ctypes.CDLL(LIB_HIP)  # loads without a GPU
    for s in declared:
        assert hasattr(lib, s)
    lib.xfthip_last_error.restype = ctypes.c_char_p
    assert isinstance(lib.xfthip_last_error(), bytes)


@pytest.mark.skipif(not os.path.exists(LIB_LAYERS), reason="host library not built")
def test_host_layer_exports_reference_entry_points(tmp_path):
    out = subprocess.check_output(["nm", "-DC", "--defined-only", LIB_LAYERS], text=True)
    for fn in ("xft::invokeLayerLLaMA(", "xft::invokeAttentionLLaMA(", "xft::invokeAttention(", "xft::invokeMLPLLaMA(", "xft::invokeGemm(",
               "xft::invokeRmsNorm(", "xft::invokeLayerNorm(", "xft::invokeRotaryEmbedding("):
        assert fn in out, fn
    # the signatures are the reference's: a translation unit written against its headers links
    src = r'''
    #include "layers_decoder.h"
    #include "layers_attention.h"
    #include "layers_mlp.h"
    #include "layers_gemm.h"
    #include "layers_norm.h"
    #include "layers_rotary_embedding.h"
    int main(int argc, char **) {
        if (argc > 100) {  // never executed: link check only
            xft::invokeLayerLLaMA(xft::DataType::bf16, xft::ActivationType::SILU, xft::NormType::RMS, 1, 1, 128, 32, 32, 8, 8,
                    0, 1, 0, 4096, 11008, nullptr, 4096, nullptr, 4096, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                    nullptr, nullptr, nullptr, nullptr, nullptr);
            xft::invokeAttentionLLaMA(xft::DataType::bf16, 1, 1, 128, 32, 32, 8, 8, 0, 1, 0, 4096, nullptr, 4096, nullptr, 4096,
                    nullptr, nullptr, nullptr, nullptr);
            xft::invokeMLPLLaMA(xft::DataType::bf16, xft::ActivationType::SILU, 1, 4096, 11008, nullptr, 4096, nullptr, 4096,
                    nullptr, nullptr, nullptr);
            xft::invokeAttention(xft::DataType::bf16, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 4096, 1024, 0.088f, 1,
                    nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, false, nullptr);
            xft::invokeGemm(xft::DataType::bf16, false, false, 1, 1, 8, 1.0f, nullptr, 8, nullptr, 0.0f, nullptr, 1);
            xft::invokeRmsNorm(xft::DataType::fp32, nullptr, nullptr, nullptr, 1, 8);
            xft::invokeLayerNorm(xft::DataType::fp32, nullptr, nullptr, nullptr, nullptr, 1, 8);
            xft::invokeRotaryEmbedding(xft::DataType::bf16, nullptr, nullptr, nullptr, nullptr, nullptr, 128, 128, 128, 1, 1,
                    128, 1);
        }
        return 0;
    }
    '''
    cpp = str(tmp_path / "link_check.cpp")
    exe = str(tmp_path / "link_check")
    open(cpp, "w").write(src)
    subprocess.check_call(["g++", "-std=c++17", "-I" + os.path.join(ROOT, "include"), cpp, "-o", exe, "-L" + PKG,
                           "-lxft_layers", "-lxft_hip", "-Wl,-rpath," + PKG])


@pytest.mark.skipif(not os.path.exists(LIB_LAYERS), reason="host library not built")
def test_host_layer_exports_the_model_classes(tmp_path):
    """xft::AutoModel / xft::Model as include/models.h declares them (the generation loop of the
    reference's examples: config, input, generate until isDone, finalize) link against the library."""
    out = subprocess.check_output(["nm", "-DC", "--defined-only", LIB_LAYERS], text=True)
    for fn in ("xft::AutoModel::AutoModel(", "xft::Model::generate()", "xft::Model::isDone()", "xft::Model::finalize()",
               "xft::Model::input(", "xft::Model::config(", "xft::Model::setStopWords(", "xft_automodel_create",
               "xft_sample_candidates"):
        assert fn in out, fn
    src = r'''
    #include "models.h"
    int main(int argc, char **argv) {
        if (argc > 100) {  // never executed: link check only
            xft::AutoModel model(argv[1], xft::DataType::int8, xft::DataType::fp16);
            std::vector<int32_t> ids = {1, 2, 3, 4};
            model.config(/*maxLen*/ 16, /*numBeams*/ 1, 1, 1.0f, false, /*eos*/ 2, /*pad*/ 0, /*doSample*/ true, 0.8f, 40, 0.9f, 1.1f,
                    {{5, 6}});
            SearcherConfig cfg(32);
            model.config(cfg);
            model.input(ids, 2);
            while (!model.isDone()) { std::vector<int32_t> next = model.generate(); (void)next; }
            std::vector<int32_t> all = model.finalize();
            return (int)all.size() + model.getVocabSize() + model.getMaxSeqLen() + model.getBatchSize() + model.getSeqLen()
                    + model.getRank() + (int)model.isMaster() + model.getConfig().maxLen;
        }
        return 0;
    }
    '''
    cpp = str(tmp_path / "model_link_check.cpp")
    exe = str(tmp_path / "model_link_check")
    open(cpp, "w").write(src)
    subprocess.check_call(["g++", "-std=c++17", "-I" + os.path.join(ROOT, "include"), cpp, "-o", exe, "-L" + PKG,
                           "-lxft_layers", "-lxft_hip", "-Wl,-rpath," + PKG])
    assert subprocess.run([exe]).returncode == 0


def test_package_refuses_to_import_without_the_library(tmp_path):
    """The Python binding has no CPU fallback: without libxft_hip.so the import raises."""
    import shutil
    pkg = tmp_path / "xfastertransformer_amd"
    pkg.mkdir()
    for f in ("__init__.py", "capi.py"):
        shutil.copy(os.path.join(PKG, f), pkg / f)
    code = "import sys; sys.path.insert(0, %r); import xfastertransformer_amd.capi" % str(tmp_path)
    r = subprocess.run(["python3", "-c", code], capture_output=True, text=True)
    assert r.returncode != 0 and "no CPU fallback" in r.stderr


@pytest.mark.skipif(not os.path.exists(LIB_LAYERS), reason="host library not built")
def test_model_header_declares_what_the_reference_declares():
    """Every public member function the reference's include/models.h declares for xft::Model (its
    lines 24-141) is declared here with the same parameter list, apart from the documented exclusions;
    all nine set_input overloads are exported."""
    ours = open(os.path.join(ROOT, "include", "models.h")).read()
    ours = re.sub(r"//[^\n]*", "", ours)
    flat = re.sub(r"\s+", " ", ours)
    # the reference's declarations, parameter lists normalised to single spaces
    want = [
        "void input(std::vector<int32_t> &inputIds_, int batchSize_);",
        "void config(SearcherConfig &config_, const std::vector<std::vector<int>> &stopWordsList_ = {});",
        "std::vector<int> set_input(std::vector<int32_t> &inputIds_, int batchSize_, int maxLen_ = -1, int numBeams_ = 1,",
        "std::vector<int> set_input(std::vector<int32_t> &inputIds_, int batchSize_, SearcherConfig &config_,",
        "std::vector<int> set_input(std::vector<std::vector<int32_t>> &inputIds_, SearcherConfig &config_,",
        "std::vector<int> set_input(std::vector<std::vector<int32_t>> &inputIds_, int maxLen_ = -1, int numBeams_ = 1,",
        "std::vector<int> set_input(std::vector<std::vector<int32_t>> &inputIds_, std::vector<int> seqIDs, SearcherConfig &config_,",
        "std::vector<int> set_input( std::vector<std::vector<int32_t>> &inputIds_, std::vector<int> seqIDs = {}, int maxLen = -1);",
        "std::vector<int> set_input( std::vector<int32_t> &inputIds_, int batchSize_, std::vector<int> seqIDs = {}, int maxLen = -1);",
        "std::vector<int> set_input( std::vector<int32_t> &inputIds_, int batchSize_, std::vector<int> seqIDs, const std::vector<int> &maxLen);",
        "std::vector<int> set_input(std::vector<int32_t> &inputIds_, std::vector<int32_t> &seqLens_, std::vector<int> seqIDs, std::vector<int> &maxLen);",
        "bool isDone();", "std::tuple<float *, int, int> forward(bool logitsAll = true);", "std::vector<int32_t> generate();",
        "void createSearcher(SearcherConfig &config_);", "void initMaxSeqLen();", "std::vector<int32_t> finalize();",
        "void setPrefix(std::vector<int32_t> &prefixIDs);", "void unsetPrefix();",
        "bool setStopWords(std::vector<std::vector<int>> stopWordsList);", "bool freeSeqs(std::vector<int> &seqIDs);",
    ]
    for decl in want:
        assert decl in flat, decl
    out = subprocess.check_output(["nm", "-D", "--defined-only", LIB_LAYERS], text=True)
    assert len([l for l in out.splitlines() if "_ZN3xft5Model9set_inputE" in l]) == 9
    assert "_ZN3xft15invokeLayerNormENS_8DataTypeEPvPKvS3_S3_iiiif" in out
