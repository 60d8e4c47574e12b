#!/usr/bin/env python3
"""Writes tests/golden/reference_extern_symbols.json: the names the reference's Rust crates
declare in `extern "C"` blocks for the EXL3 linear path (read as text from the reference
tree; run in the build container, where /root/reference exists).  tests/test_abi.py holds
the library's exported symbols against this list."""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
FILES = ["crates/berth-kernels/src/ffi.rs", "crates/berth-kernels/src/prefill_lin.rs", "crates/berth-kernels/src/ops.rs"]


def blocks(text):
    """(is_test_only, body) for every `unsafe extern "C" { ... }` block."""
    for m in re.finditer(r'((?:#\[cfg\(test\)\]\s*)?)unsafe extern "C" \{', text):
        depth, i = 1, m.end()
        while depth:
            depth += {"{": 1, "}": -1}.get(text[i], 0)
            i += 1
        yield bool(m.group(1)), text[m.end():i - 1]


out = {}
for rel in FILES:
    text = open(os.path.join(REF, rel)).read()
    entry = {"always": [], "test_only": []}
    for test_only, body in blocks(text):
        names = re.findall(r"\bfn (berth_[a-z0-9_]+)\s*\(", body)
        entry["test_only" if test_only else "always"] += names
    out[rel] = entry
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_extern_symbols.json")
json.dump(out, open(path, "w"), indent=1, sort_keys=True)
print(path, {k: (len(v["always"]), len(v["test_only"])) for k, v in out.items()})
