"""Reads the virtual-method table of a C++ class out of a header (text only, nothing is compiled): name, return type,
parameter types, constness and whether the method is pure. Used to compare this build's LlmExecutorBase with the
method list of the reference's runtime/executor/llm_executor_base.h:32-119 (kept as tests/golden/llm_executor_base_methods.json)."""
from __future__ import annotations

import re

# spelling differences that are stand-in types, not interface differences
_ALIASES = [("::litert::", ""), ("litert::", ""), ("absl::", ""), ("std::", "")]


def _norm_type(t: str) -> str:
    for a, b in _ALIASES:
        t = t.replace(a, b)
    t = re.sub(r"\s+", " ", t).strip()
    return re.sub(r"\s*([&*<>,])\s*", r"\1", t)


def _split_args(args: str):
    out, depth, cur = [], 0, ""
    for ch in args:
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur)
    return out


def _param_type(p: str) -> str:
    p = p.split("=")[0].strip()
    m = re.match(r"^(.*?[&*\s>])\s*(\w+)$", p)  # drop the parameter name
    return _norm_type(m.group(1) if m else p)


def virtual_methods(header_text: str, class_name: str):
    text = re.sub(r"//[^\n]*", "", header_text)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    m = re.search(r"class\s+%s\b[^{;]*\{" % re.escape(class_name), text)
    if not m:
        raise ValueError(f"class {class_name} not found")
    depth, i = 1, m.end()
    while depth and i < len(text):
        depth += {"{": 1, "}": -1}.get(text[i], 0)
        i += 1
    body = text[m.end():i]
    methods = []
    pat = re.compile(r"virtual\s+(?P<ret>[^();{}]+?)\s*\b(?P<name>~?\w+)\s*\((?P<args>[^)]*)\)\s*(?P<const>const)?\s*(?P<tail>=\s*0|=\s*default|\{|;)")
    for f in pat.finditer(body):
        if "~" in f.group("ret") or f.group("name").startswith("~"):  # the destructor
            continue
        methods.append({
            "name": f.group("name"),
            "returns": _norm_type(f.group("ret")),
            "params": [_param_type(a) for a in _split_args(f.group("args"))],
            "const": bool(f.group("const")),
            "pure": f.group("tail").replace(" ", "") == "=0",
        })
    return methods
