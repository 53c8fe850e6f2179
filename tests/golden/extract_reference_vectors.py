#!/usr/bin/env python3
"""Transcribes the known-answer vectors of the reference's own kernel unit tests into JSON.

The reference's tests (test/runtime/local/kernels/*.cpp in the reference checkout) define their
inputs and expected outputs as literal matrices (`genGivenVals<DT>(numRows, {v0, v1, ...})`) and
check them with calls such as `checkEwBinaryMat(BinaryOpCode::ADD, m1, m2, m3)`. This script reads
those files AS TEXT (nothing of the reference is compiled, imported or executed), and writes per
file: every test case, its literal matrices and its check calls. The JSON holds data only.

    python tests/golden/extract_reference_vectors.py /root/reference

The output (tests/golden/reference_kernel_tests.json) is committed; the parity tests read it and
never need the reference checkout.
"""
from __future__ import annotations

import json
import re
import sys
from pathlib import Path

FILES = [
    "EwBinaryMatTest.cpp", "EwBinaryObjScaTest.cpp", "EwUnaryMatTest.cpp", "AggAllTest.cpp", "AggRowTest.cpp",
    "AggColTest.cpp", "MatMulTest.cpp", "SyrkTest.cpp", "SolveTest.cpp", "SoftmaxTest.cpp",
    "DNNConv2DForwardTest.cpp", "DNNPoolingTestForward.cpp", "DNNBiasAddForwardTest.cpp",
    "DNNBatchNorm2DForwardTest.cpp", "CUDA/MatMulTest.cpp", "CUDA/DNNAffineTest.cpp", "CUDA/BiasAddTest.cpp",
    "CUDA/DNNBatchNormTest.cpp", "CUDA/DNNConvolutionTest.cpp", "CUDA/DNNSoftmaxTest.cpp",
    "CUDA/DNNActivationTest.cpp", "CUDA/DNNPoolingTest.cpp", "TransposeTest.cpp", "ColBindTest.cpp",
    "ExtractColTest.cpp", "DNNConv2DBackwardTest.cpp", "DNNPoolingBackwardTest.cpp", "DNNBatchNorm2DBackwardTest.cpp",
]

NUM = re.compile(r"^[-+]?(\d+\.?\d*|\.\d+)([eE][-+]?\d+)?[fFlL]?$")


def parse_value(tok: str):
    """One literal of a genGivenVals list -> float, or None if it is not a plain number."""
    t = tok.strip()
    if not t:
        return "skip"
    t = re.sub(r"^\(?\s*(?:typename\s+)?(?:VT|VTRes|VTArg|DT::VT|typename DT::VT|double|float|size_t|int64_t)\s*\)\s*", "", t)
    m = re.match(r"^(?:VT|VTRes|VTArg|double|float)\((.*)\)$", t)
    if m:
        t = m.group(1).strip()
    sign = 1.0
    while t.startswith("-") and not NUM.match(t):
        sign, t = -sign, t[1:].strip()
    low = t.lower()
    if "quiet_nan" in low or low in ("nan", "nan_val"):
        return float("nan")
    if "infinity" in low or low == "inf":
        return sign * float("inf")
    if "denorm_min" in low:
        return "denorm_min" if sign > 0 else None  # the value type's smallest subnormal, resolved at replay
    if NUM.match(t):
        return sign * float(t.rstrip("fFlL"))
    return None


def split_top(s: str) -> list[str]:
    """Splits at commas that are not nested in (), {}, <>."""
    out, depth, cur = [], 0, []
    for ch in s:
        if ch in "({<":
            depth += 1
        elif ch in ")}>":
            depth -= 1
        if ch == "," and depth == 0:
            out.append("".join(cur))
            cur = []
        else:
            cur.append(ch)
    if "".join(cur).strip():
        out.append("".join(cur))
    return [a.strip() for a in out]


def extract(path: Path) -> dict:
    src = path.read_text().replace("\\\n", " ")  # join macro continuation lines
    src = re.sub(r"//[^\n]*", "", src)
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    defines = dict(re.findall(r"#define\s+(\w+)\s+([^\n]+)", src))
    flat = re.sub(r"\s+", " ", src)
    # test-case boundaries
    heads = list(re.finditer(r"(TEMPLATE_PRODUCT_TEST_CASE|TEMPLATE_TEST_CASE|TEST_CASE)\(", flat))
    cases = []
    for i, h in enumerate(heads):
        body = flat[h.end():heads[i + 1].start() if i + 1 < len(heads) else len(flat)]
        header = body[:body.index("{")] if "{" in body else body[:200]
        name_m = re.search(r'"([^"]*)"', header)
        types = header
        for k, v in defines.items():
            types = types.replace(k, v)
        case = {"name": name_m.group(1) if name_m else "", "header": header.strip()[:200], "types": types.strip()[:300],
                "matrices": {}, "checks": []}
        for m in re.finditer(r"(?:auto|DT \*|DTArg \*|DTRes \*|DenseMatrix<\w+> \*|DT\*)?\s*(\w+)\s*=\s*genGivenVals<([^>]*(?:<[^>]*>)?)>\(\s*(\d+)\s*,\s*\{([^}]*)\}\s*\)", body):
            var, dtype, rows, vals = m.group(1), m.group(2), int(m.group(3)), m.group(4)
            parsed = [parse_value(t) for t in split_top(vals)]
            parsed = [p for p in parsed if p != "skip"]
            if any(p is None for p in parsed):
                continue  # strings or expressions: not a numeric matrix
            # a name may be defined several times (per SECTION, or per value-type branch): keep all,
            # with their position, so that a check can take the definition that precedes it
            case["matrices"].setdefault(var, []).append({"pos": m.start(), "rows": rows, "values": parsed})
        # views made with the slicing kernels: `sliceRow(res, arg, lower, upper, ctx)` / `sliceCol(...)`
        for m in re.finditer(r"\bslice(Row|Col)\(\s*(\w+)\s*,\s*(\w+)\s*,\s*(\d+)\s*,\s*(\d+)\s*,", body):
            case.setdefault("slices", {})[m.group(2)] = {"of": m.group(3), "axis": m.group(1).lower(), "lo": int(m.group(4)),
                                                         "hi": int(m.group(5)), "pos": m.start()}
        for m in re.finditer(r"\b(check\w+)\s*(?:<[^>(]*>)?\(([^;]*?)\);", body):
            case["checks"].append({"fn": m.group(1), "args": split_top(m.group(2)), "pos": m.start()})
        for m in re.finditer(r"(CHECK_THROWS|REQUIRE_THROWS_AS|CHECK_THROWS_AS|REQUIRE_THROWS)\((.*?)\);", body):
            case["checks"].append({"fn": m.group(1), "args": [m.group(2)[:200]], "pos": m.start()})
        # the argument lists of direct kernel calls (DNN tests call apply(...) inside a helper)
        for m in re.finditer(r"(\w+(?:::\w+)*(?:<[^;(]*>)?::apply)\(([^;]*?)\);", body):
            case["checks"].append({"fn": m.group(1), "args": split_top(m.group(2)), "pos": m.start()})
        if case["matrices"] or case["checks"]:
            cases.append(case)
    # helper functions before the first test case (they carry the fixed kernel parameters)
    pre = flat[:heads[0].start()] if heads else flat
    helpers = [{"fn": m.group(1), "args": split_top(m.group(2))}
               for m in re.finditer(r"(\w+(?:::\w+)*(?:<[^;(]*>)?::apply)\(([^;]*?)\);", pre)]
    # input generators shared by several test cases: `DT *genInput() { return genGivenVals<DT>(2, {...}); }`
    helper_mats = {}
    for m in re.finditer(r"(\w+)\(\)\s*\{\s*return genGivenVals<[^>]*>\(\s*(\d+)\s*,\s*\{([^}]*)\}\s*\)", pre):
        vals = [parse_value(t) for t in split_top(m.group(3))]
        vals = [v for v in vals if v != "skip"]
        if all(v is not None for v in vals):
            helper_mats[m.group(1)] = {"rows": int(m.group(2)), "values": vals}
    return {"file": str(path.name if "CUDA" not in str(path) else "CUDA/" + path.name), "helper_calls": helpers,
            "helper_matrices": helper_mats, "cases": cases}


def main() -> int:
    ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    base = ref / "test" / "runtime" / "local" / "kernels"
    out = [extract(base / f) for f in FILES if (base / f).exists()]
    dst = Path(__file__).resolve().parent / "reference_kernel_tests.json"

    def clean(o):
        if isinstance(o, float):
            if o != o:
                return "nan"
            if o in (float("inf"), float("-inf")):
                return "inf" if o > 0 else "-inf"
        if isinstance(o, list):
            return [clean(x) for x in o]
        if isinstance(o, dict):
            return {k: clean(v) for k, v in o.items()}
        return o

    dst.write_text(json.dumps(clean(out), indent=1))
    n_m = sum(len(v) for f in out for c in f["cases"] for v in c["matrices"].values())
    n_c = sum(len(c["checks"]) for f in out for c in f["cases"])
    print(f"wrote {dst}: {len(out)} files, {sum(len(f['cases']) for f in out)} test cases, {n_m} matrices, {n_c} checks")
    return 0


if __name__ == "__main__":
    sys.exit(main())
