#!/usr/bin/env python3
"""Writes tests/golden/c_ext_signatures.json: the argument names, their order and
their defaults of the reference's Python operators on the GPU<->CPU transfer path,
read from the `py::arg(...)` lists of the reference's pybind module.

    python tests/golden/make_signatures.py [/root/reference]

The reference file is read as text; nothing of it is imported or executed.  The
fixture is data only: per operator a list of [name, default] pairs in declaration
order, where default is {"required": true} or {"value": ...} for plain literals
(bool, int, string) and {"empty": "tensor" | "list" | "map"} for the empty
containers the reference spells `torch::empty({0})`, `std::vector<...>()` and
`std::map<...>()`.  tests/test_signatures.py holds flexkv_amd.c_ext to it.
"""
from __future__ import annotations

import json
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))

# (python name in the module, what the test compares it with)
WANTED = {
    "transfer_kv_blocks",
    "transfer_kv_blocks_ssd",
    "TPTransferThreadGroup.__init__",
    "TPTransferThreadGroup.update_gpu_block_ptrs",
    "TPTransferThreadGroup.tp_group_transfer",
    "LayerwiseTransferGroup.__init__",
    "LayerwiseTransferGroup.init_swa_multi_group",
    "LayerwiseTransferGroup.layerwise_transfer",
    "LayerwiseTransferGroup.layerwise_transfer_multi_group",
}

OPEN, CLOSE = "([{", ")]}"


def matching_paren(text: str, start: int) -> int:
    """Index of the parenthesis that closes text[start] == '('; string literals and
    comments are skipped."""
    depth, i, n = 0, start, len(text)
    while i < n:
        c = text[i]
        if c == '"':
            i += 1
            while text[i] != '"':
                i += 2 if text[i] == "\\" else 1
        elif text.startswith("//", i):
            i = text.index("\n", i)
        elif c in OPEN:
            depth += 1
        elif c in CLOSE:
            depth -= 1
            if depth == 0:
                return i
        i += 1
    raise ValueError("unbalanced parentheses")


def default_expression(body: str, at: int) -> tuple[str, int]:
    """The expression behind '=' at body[at], up to the next comma at nesting depth 0
    or the end of the argument list (angle brackets of template arguments count as
    nesting)."""
    depth, i = 0, at
    while i < len(body):
        c = body[i]
        if c == '"':
            i += 1
            while body[i] != '"':
                i += 2 if body[i] == "\\" else 1
        elif c in OPEN or c == "<":
            depth += 1
        elif c in CLOSE or c == ">":
            if depth == 0:   # the parenthesis that closes the whole .def(...)
                break
            depth -= 1
        elif c == "," and depth == 0:
            break
        i += 1
    return body[at:i].strip(), i


def literal(expr: str):
    expr = " ".join(expr.split())
    if expr in ("true", "false"):
        return {"value": expr == "true"}
    if re.fullmatch(r"-?\d+", expr):
        return {"value": int(expr)}
    if re.fullmatch(r'"[^"]*"', expr):
        return {"value": expr[1:-1]}
    if expr.startswith("torch::empty("):
        return {"empty": "tensor"}
    if expr.startswith("std::vector<") and expr.endswith("()"):
        return {"empty": "list"}
    if expr.startswith("std::map<") and expr.endswith("()"):
        return {"empty": "map"}
    if expr in ("nullptr", "py::none()"):
        return {"value": None}
    return {"expression": expr}   # kept as written; none of the operators compared uses one


def arguments(body: str):
    out = []
    for m in re.finditer(r'py::arg\(\s*"(\w+)"\s*\)', body):
        i = m.end()
        while i < len(body) and body[i].isspace():
            i += 1
        if i < len(body) and body[i] == "=":
            expr, _ = default_expression(body, i + 1)
            out.append([m.group(1), literal(expr)])
        else:
            out.append([m.group(1), {"required": True}])
    return out


def parse(text: str):
    """Every m.def("name", ...) and every .def(...) of a py::class_ in order of
    appearance: {qualified name: [argument lists]} (a class can have several inits)."""
    events = []
    for m in re.finditer(r'py::class_<[^;]*?\(\s*m\s*,\s*"(\w+)"', text, re.S):
        events.append((m.start(), "class", m.group(1), None))
    for m in re.finditer(r'\bm\.def\(\s*"(\w+)"', text):
        events.append((m.start(), "mdef", m.group(1), text.index("(", m.start())))
    for m in re.finditer(r'(?<![\w.])\.def\(\s*(?:"(\w+)"|py::init)', text):
        events.append((m.start(), "def", m.group(1) or "__init__", text.index("(", m.start())))
    events.sort()
    found, cls = {}, None
    for _, kind, name, paren in events:
        if kind == "class":
            cls = name
            continue
        body = text[paren:matching_paren(text, paren) + 1]
        key = name if kind == "mdef" else f"{cls}.{name}"
        found.setdefault(key, []).append(arguments(body))
    return found


def main() -> None:
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    path = os.path.join(ref, "csrc", "bindings.cpp")
    with open(path, encoding="utf-8") as f:
        found = parse(f.read())
    missing = sorted(WANTED - set(found))
    if missing:
        raise SystemExit(f"not found in {path}: {missing}")
    out = {"source": "csrc/bindings.cpp (py::arg lists; names, order, defaults)",
           "operators": {k: found[k] for k in sorted(WANTED)}}
    dst = os.path.join(HERE, "c_ext_signatures.json")
    with open(dst, "w", encoding="utf-8") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    for k in sorted(WANTED):
        print(k, [len(a) for a in found[k]])


if __name__ == "__main__":
    main()
