"""Extracts the literals of the reference's conv2d tests into conv2d_literals.json.

Reads dfdx-core/src/tensor_ops/conv2d/tests.rs as text (nothing is compiled or run): for every test that spells
out its tensors, the input, filter and bias literals, the (stride, padding, dilation, groups) constants, the
asserted output and the asserted gradients.  Tests built on seeded random tensors hold no usable literals and
are skipped.  Usage: python tests/golden/make_conv2d_literals.py [path-to-reference-checkout]
"""
import ast
import json
import os
import re
import sys

ROOT = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
SRC = os.path.join(ROOT, "dfdx-core/src/tensor_ops/conv2d/tests.rs")


def matching(text, start):
    """Index just past the bracket that closes the one at text[start]."""
    pairs = {"(": ")", "[": "]"}
    close = pairs[text[start]]
    depth = 0
    for i in range(start, len(text)):
        if text[i] == text[start]:
            depth += 1
        elif text[i] == close:
            depth -= 1
            if depth == 0:
                return i + 1
    raise ValueError("unbalanced")


def literal(text):
    return ast.literal_eval(text.strip())


def main():
    src = open(SRC).read()
    lines = src.split("\n")
    starts = [(m.start(), m.group(1)) for m in re.finditer(r"fn (test_\w+)\(\)", src)]
    cases = []
    for idx, (pos, name) in enumerate(starts):
        end = starts[idx + 1][0] if idx + 1 < len(starts) else len(src)
        body = src[pos:end]
        body = re.sub(r"//[^\n]*", "", body)
        tensors = {}
        for m in re.finditer(r"let (\w+)\s*=\s*dev\s*\.tensor\(", body):
            stop = matching(body, m.end() - 1)
            tensors[m.group(1)] = literal(body[m.end():stop - 1])
        conv = re.search(r"\.conv2d\(\s*Const::<(\d+)>,\s*Const::<(\d+)>,\s*Const::<(\d+)>,\s*Const::<(\d+)>,?\s*\)", body)
        asserts = {}
        for m in re.finditer(r"assert_close_to_literal!\(", body):
            stop = matching(body, m.end() - 1)
            inner = body[m.end():stop - 1]
            expr, lit = inner.split(",", 1)
            asserts[re.sub(r"\s+", "", expr)] = literal(lit)
        x = tensors.get("x")
        w = tensors.get("weight", tensors.get("w"))
        if x is None or w is None or conv is None:
            continue  # seeded-random test: no literals to take
        out_key = "result" if "result" in asserts else "y"
        gname = "g" if any(k.startswith("g.get") for k in asserts) else "grads"
        wname = "weight" if "weight" in tensors else "w"
        loss = "exp_mean" if re.search(r"\.exp\(\)\s*\.mean\(\)\s*\.backward", body) else "mean"
        line0 = src[:pos].count("\n") + 1
        case = {
            "name": name, "ref": f"conv2d/tests.rs:{line0}-{line0 + body.rstrip().count(chr(10))}",
            "stride": int(conv.group(1)), "padding": int(conv.group(2)), "dilation": int(conv.group(3)),
            "groups": int(conv.group(4)), "x": x, "weight": w, "out": asserts[out_key], "loss": loss,
            "grad_x": asserts[f"{gname}.get(&x)"], "grad_weight": asserts[f"{gname}.get(&{wname})"],
        }
        if "bias" in tensors:
            case["bias"] = tensors["bias"]
            case["grad_bias"] = asserts[f"{gname}.get(&bias)"]
        cases.append(case)
    doc = {"_source": "Literals of dfdx-core/src/tensor_ops/conv2d/tests.rs (PyTorch-produced, see the doc comments "
                      "there), extracted by tests/golden/make_conv2d_literals.py.  x is (C, H, W), weight "
                      "(O, C/groups, K, K); out = conv2d(x, weight) + bias broadcast over (H_out, W_out).",
           "cases": cases}
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "conv2d_literals.json")
    json.dump(doc, open(dst, "w"), indent=1)
    print("wrote", dst, [c["name"] for c in cases])
    del lines


if __name__ == "__main__":
    main()
