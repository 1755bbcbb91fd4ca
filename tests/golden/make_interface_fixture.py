"""Writes tests/golden/llm_executor_base_methods.json: the virtual-method list (names, return and parameter types with
namespace qualifiers dropped, constness, purity) of LlmExecutorBase as the reference declares it in
runtime/executor/llm_executor_base.h. The header is read as text; nothing of the reference is imported or run.

    python tests/golden/make_interface_fixture.py [/root/reference]
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from cpp_interface import virtual_methods  # noqa: E402

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
src = "runtime/executor/llm_executor_base.h"
with open(os.path.join(ref, src)) as f:
    methods = virtual_methods(f.read(), "LlmExecutorBase")
with open(os.path.join(HERE, "llm_executor_base_methods.json"), "w") as f:
    json.dump({"source": src, "class": "LlmExecutorBase", "methods": methods}, f, indent=1)
    f.write("\n")
print(len(methods), "methods")
