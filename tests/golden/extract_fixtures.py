#!/usr/bin/env python3
"""Transcribe the tensor literals held by the reference's own unit tests into JSON fixtures.

The reference keeps its ground truth as `Tensor::new([...])` literals inside `#[cfg(test)]`
modules (4-decimal values its authors produced offline with PyTorch).  This script reads the
reference sources as text, finds every `#[test] fn`, and for each `let NAME = Tensor::new(<literal>)`
inside it records the nested-list literal under  file -> test function -> NAME  (a repeated NAME
gets a numeric suffix).  Only data is extracted; no reference code is kept.

Run in the build container (needs /root/reference):
    python tests/golden/extract_fixtures.py
It rewrites tests/golden/reference_literals.json.
"""
import ast
import json
import os
import re
import sys

REF = os.environ.get("SAGE_REFERENCE", "/root/reference")
FILES = [
    "src/ops/map.rs", "src/ops/core.rs", "src/ops/reduce.rs", "src/ops/gemm.rs",
    "src/ops/conv.rs", "src/ops/nn.rs", "src/layers.rs", "src/shape.rs",
]

TEST_RE = re.compile(r"#\[test\]\s*(?:pub\s+)?fn\s+(\w+)\s*\(")
LET_RE = re.compile(r"let\s+(?:mut\s+)?(\w+)\s*=\s*Tensor::new\(")


def balanced(text, start, open_ch, close_ch):
    """Return index one past the bracket that closes text[start] (== open_ch)."""
    depth = 0
    i = start
    while i < len(text):
        c = text[i]
        if c == open_ch:
            depth += 1
        elif c == close_ch:
            depth -= 1
            if depth == 0:
                return i + 1
        i += 1
    raise ValueError("unbalanced")


def strip_comments(src):
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return "\n".join(line.split("//")[0] for line in src.splitlines())


def parse_literal(lit):
    lit = re.sub(r"(\d)_?(f32|u32|i32|usize)\b", r"\1", lit)
    lit = re.sub(r"(\d)\.(?=[,\]\s])", r"\1.0", lit)
    return ast.literal_eval(lit)


def shape_of(v):
    s = []
    while isinstance(v, list):
        s.append(len(v))
        v = v[0]
    return s


def main():
    out = {}
    for rel in FILES:
        src = strip_comments(open(os.path.join(REF, rel)).read())
        tests = {}
        for m in TEST_RE.finditer(src):
            name = m.group(1)
            brace = src.index("{", m.end())
            end = balanced(src, brace, "{", "}")
            body = src[brace:end]
            vals = {}
            for lm in LET_RE.finditer(body):
                var = lm.group(1)
                p = lm.end() - 1
                pend = balanced(body, p, "(", ")")
                arg = body[p + 1:pend - 1].strip()
                if not arg.startswith("["):
                    continue
                try:
                    data = parse_literal(arg)
                except Exception as e:  # literal that is not plain data
                    print(f"skip {rel}:{name}:{var}: {e}", file=sys.stderr)
                    continue
                key, n = var, 1
                while key in vals:
                    n += 1
                    key = f"{var}#{n}"
                vals[key] = {"shape": shape_of(data), "data": data}
            if vals:
                tests[name] = vals
        out[rel] = tests
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_literals.json")
    with open(dst, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    for rel, tests in out.items():
        for t, vals in tests.items():
            print(rel, t, {k: v["shape"] for k, v in vals.items()})


if __name__ == "__main__":
    main()
