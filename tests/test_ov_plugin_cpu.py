"""The OpenVINO adapter under src/ov_plugin compiles against the plugin API headers of an OpenVINO 2021.4 tree
(`make -C src/ov_plugin syntax`).  Skipped where no such tree is present."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PLUGIN = os.path.join(ROOT, "src", "ov_plugin")
OPENVINO = os.environ.get("OPENVINO", "/root/reference")

SOURCES = ["function_to_graph.cpp", "hip_infer_request.cpp", "hip_async_infer_request.cpp", "hip_executable_network.cpp",
           "hip_plugin.cpp"]


def test_sources_are_present_and_bind_only_declared_symbols():
    """every hipie_* name the adapter uses is declared in include/hipie.h"""
    import re
    with open(os.path.join(ROOT, "include", "hipie.h")) as f:
        header = f.read()
    declared = set(re.findall(r"\b(hipie_[a-z0-9_]+)\s*\(", header)) | set(re.findall(r"\b(hipie_[a-z0-9_]+)\b", header))
    for name in SOURCES + ["hip_common.hpp", "function_to_graph.hpp", "hip_plugin.hpp", "hip_executable_network.hpp",
                           "hip_infer_request.hpp", "hip_async_infer_request.hpp"]:
        with open(os.path.join(PLUGIN, name)) as f:
            text = f.read()
        used = {u for u in re.findall(r"\b(hipie_[a-z0-9_]+)\b", text) if not u.endswith("_")}   # "hipie_graph_*" in prose
        assert used <= declared, (name, sorted(used - declared))
    with open(os.path.join(PLUGIN, "hip_plugin.cpp")) as f:
        assert "IE_DEFINE_PLUGIN_CREATE_FUNCTION" in f.read()


@pytest.mark.skipif(not os.path.isdir(os.path.join(OPENVINO, "inference-engine", "src", "plugin_api")),
                    reason="no OpenVINO source tree to check against")
def test_adapter_passes_syntax_check_against_plugin_api():
    r = subprocess.run(["make", "-C", PLUGIN, "syntax", "OPENVINO=" + OPENVINO], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "syntax ok" in r.stdout
