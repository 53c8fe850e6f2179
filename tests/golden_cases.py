"""Replays the reference's own kernel unit tests (tests/golden/reference_kernel_tests.json, written
by tests/golden/extract_reference_vectors.py) against a backend: the CPU oracle or the HIP kernels.

Every check call of the reference's tests is mapped onto the backend's kernel of the same name; the
comparison is the one the reference's test uses (operator== -> exact; checkEqApprox -> its epsilon).
"""
from __future__ import annotations

import json
import re
from pathlib import Path

import numpy as np

GOLDEN = Path(__file__).resolve().parent / "golden" / "reference_kernel_tests.json"

BIN = {n: i for i, n in enumerate(["ADD", "SUB", "MUL", "DIV", "POW", "MOD", "LOG", "EQ", "NEQ", "LT", "LE", "GT", "GE",
                                   "MIN", "MAX", "AND", "OR", "BITWISE_AND", "CONCAT"])}
UN = {n: i for i, n in enumerate(["MINUS", "ABS", "SIGN", "SQRT", "EXP", "LN", "SIN", "COS", "TAN", "ASIN", "ACOS",
                                  "ATAN", "SINH", "COSH", "TANH", "FLOOR", "CEIL", "ROUND", "ISNAN", "UPPER", "LOWER"])}
AGG = {n: i for i, n in enumerate(["SUM", "PROD", "MIN", "MAX", "IDXMIN", "IDXMAX", "MEAN", "STDDEV", "VAR"])}


class Skip(Exception):
    pass


class DomainError(Exception):
    pass


class KernelError(Exception):
    pass


class OutOfRange(KernelError):
    pass


def load():
    return json.loads(GOLDEN.read_text())


def _num(v):
    return {"nan": np.nan, "inf": np.inf, "-inf": -np.inf}.get(v, v) if isinstance(v, str) else v


def matrix(spec, dt):
    if "denorm_min" in spec["values"]:
        if np.dtype(dt).kind != "f":
            raise Skip("floating-point literal")
        tiny = float(np.finfo(dt).smallest_subnormal)
        spec = {**spec, "values": [tiny if v == "denorm_min" else v for v in spec["values"]]}
    vals = np.array([_num(v) for v in spec["values"]], dtype=np.float64)
    rows = spec["rows"]
    if rows == 0 or vals.size % rows:
        raise Skip("ragged literal")
    dt = np.dtype(dt)
    if dt.kind in "iu":
        # the same literals serve the reference's integer instantiations where every value is an integer of that type
        info = np.iinfo(dt)
        if not np.all(np.isfinite(vals)) or np.any(vals != np.trunc(vals)) or vals.min(initial=0) < info.min or \
                vals.max(initial=0) > min(info.max, 2 ** 53):
            raise Skip(f"literal not representable as {dt}")
    return np.ascontiguousarray(vals.reshape(rows, vals.size // rows).astype(dt))


def _scalar(tok):
    t = re.sub(r"\(\s*(typename\s+)?[\w:]+\s*\)", "", tok).strip()
    m = re.match(r"^\w+\((.*)\)$", t)
    if m:
        t = m.group(1)
    try:
        return float(t.rstrip("fFlL"))
    except ValueError:
        raise Skip(f"scalar {tok!r}")


def _ints(args):
    out = []
    for a in ",".join(args).split(","):
        if re.fullmatch(r"\d+", a.strip()):
            out.append(int(a))
    return out


def all_checks():
    """Yields (id, file, case, check) for every replayable check call."""
    for f in load():
        for ci, c in enumerate(f["cases"]):
            for ki, k in enumerate(c["checks"]):
                yield f"{f['file']}::{c['name'].strip() or ci}::{ki}:{k['fn']}", f, c, k
            if not c["checks"]:
                yield f"{f['file']}::{c['name'].strip() or ci}::direct", f, c, {"fn": "direct", "args": []}


def _eq(got, exp):
    got, exp = np.asarray(got, dtype=np.float64), np.asarray(exp, dtype=np.float64)
    assert got.shape == exp.shape, (got.shape, exp.shape)
    same = (got == exp) | (np.isnan(got) & np.isnan(exp))
    assert same.all(), f"got {got.ravel()[:12]} expected {exp.ravel()[:12]}"


def _approx(got, exp, eps):
    got, exp = np.asarray(got, dtype=np.float64), np.asarray(exp, dtype=np.float64)
    assert got.shape == exp.shape, (got.shape, exp.shape)
    both_nan = np.isnan(got) & np.isnan(exp)
    both_inf = np.isinf(exp) & (got == exp)
    ok = both_nan | both_inf | (np.abs(got - exp) <= eps)
    assert ok.all(), f"got {got.ravel()[:12]} expected {exp.ravel()[:12]} eps {eps}"


def run(backend, f, c, k, dt):
    """Replays one check; raises Skip for what is outside the float/double dense path."""
    fn, args, file = k["fn"], k["args"], f["file"]
    # a literal may be re-defined inside a test case (per SECTION / per value-type branch): a check
    # uses the definition that precedes it in the source, else the first one
    pos = k.get("pos", 1 << 60)
    mats = dict(f.get("helper_matrices", {}))
    for name, defs in c["matrices"].items():
        before = [d for d in defs if d["pos"] < pos]
        mats[name] = before[-1] if before else defs[0]
    feps = 1e-5 if dt == np.float32 else 1e-9
    is_int = np.dtype(dt).kind in "iu"
    if is_int:
        # integer instantiations: elementwise binary for si64 / ui64 / si32 / ui32, the rest for si64 only
        ew = fn in ("checkEwBinaryMat", "checkEwBinaryObjSca")
        other = fn in ("checkAggAll", "checkAggRow", "checkAggCol", "checkTranspose") or \
            (fn == "direct" and file.endswith("ColBindTest.cpp"))
        if not (ew or (other and np.dtype(dt) == np.int64)):
            raise Skip("kernel has no instantiation for this integer type on the device")

    slices = c.get("slices", {})

    def M(name):
        name = name.strip()
        if name in slices and name not in mats:
            # a view made by sliceRow / sliceCol: stays a view (of the literal's array) down to the kernel
            s = slices[name]
            base = M(s["of"])
            return base[s["lo"]:s["hi"], :] if s["axis"] == "row" else base[:, s["lo"]:s["hi"]]
        if name not in mats:
            if name in ("inputs",) and "genInput" in mats:
                return matrix(mats["genInput"], dt)
            raise Skip(f"matrix {name} is not a numeric literal")
        return matrix(mats[name], dt)

    def code(tok, table):
        name = tok.split("::")[-1].strip()
        if name not in table:
            raise Skip(f"op {tok}")
        return table[name]

    if fn in ("checkEwBinaryMat",):
        op = code(args[0], BIN)
        if op >= 17:
            raise Skip("integer/string op")
        _eq(backend.ew_binary(op, M(args[1]), M(args[2])), M(args[3]))
    elif fn == "checkEwBinaryObjSca":
        op = code(args[0], BIN)
        if op >= 17:
            raise Skip("integer/string op")
        sca = _scalar(args[2])
        if is_int:
            if sca != int(sca) or (sca < 0 and np.dtype(dt).kind == "u"):
                raise Skip("scalar not representable in the integer type")
            sca = int(sca)
        _eq(backend.ew_binary_sca(op, M(args[1]), sca), M(args[3]))
    elif fn == "checkEwUnaryMat":
        op = code(args[0], UN)
        if op >= 19:
            raise Skip("string op")
        _eq(backend.ew_unary(op, M(args[1])), M(args[2]))
    elif fn == "checkEwUnaryMatApprox":
        _approx(backend.ew_unary(code(args[0], UN), M(args[1])), M(args[2]), 1e-2)  # EwUnaryMatTest.cpp: checkEqApprox(..., 1e-2)
    elif fn == "checkEwUnaryMatThrow":
        try:
            backend.ew_unary(code(args[0], UN), M(args[1]))
        except DomainError:
            return
        raise AssertionError("expected std::domain_error")
    elif fn == "CHECK_THROWS" and "999" in args[0]:
        a = M("arg") if "arg" in mats else M(next(iter(mats)))
        try:
            if "UnaryOpCode" in args[0]:
                backend.ew_unary(999, a)
            elif "ObjSca" in args[0]:
                backend.ew_binary_sca(999, a, 1.0)
            else:
                backend.ew_binary(999, a, a)
        except KernelError:
            return
        raise AssertionError("expected an exception for op code 999")
    elif fn == "checkAggAll":
        op = code(args[0], AGG)
        if is_int and op >= 6:
            raise Skip("integer MEAN / STDDEV / VAR stay on the CPU")
        exp = _scalar(args[2])
        got = backend.agg_all(op, M(args[1]))
        _approx(np.array([got]), np.array([exp]), max(feps, abs(exp) * (1e-6 if dt == np.float32 else 1e-14)))
    elif fn in ("checkAggRow", "checkAggCol"):
        op = code(args[0], AGG)
        if is_int and op >= 6:
            raise Skip("integer MEAN / STDDEV / VAR stay on the CPU")
        got = (backend.agg_row if fn == "checkAggRow" else backend.agg_col)(op, M(args[1]))
        exp = M(args[2])
        if op in (AGG["IDXMIN"], AGG["IDXMAX"]):
            _eq(got.astype(np.float64), exp)
        else:
            _approx(got, exp, 1e-5)  # AggRowTest.cpp / AggColTest.cpp: checkEqApprox(..., 1e-5)
    elif fn in ("checkMatMul", "checkMatMulCUDA"):
        flags = [a.strip() for a in args[3:] if a.strip() in ("true", "false")]
        ta = flags[0] == "true" if flags else False
        tb = flags[1] == "true" if len(flags) > 1 else False
        _eq(backend.matmul(M(args[0]), M(args[1]), ta, tb), M(args[2]))
    elif fn == "checkSyrk":
        m = M(args[0])
        # SyrkTest.cpp:32-58: syrk(m) must equal matMul(t(m), m)
        _eq(backend.syrk(m, True), backend.matmul(m, m, True, False))
        _eq(backend.syrk(m, True), (m.astype(np.float64).T @ m.astype(np.float64)).astype(dt))
    elif fn == "checkSolve":
        # SolveTest.cpp:42-68: normal equations of X w = y, solved for w (eps 1e-6 ... 1e-4 for float)
        X, w = M("X"), M("w")
        y = backend.matmul(X, w, False, False)
        A = backend.matmul(X, X, True, False)
        b = backend.matmul(X, y, True, False)
        _approx(backend.solve(A, b), w, 1e-3 if dt == np.float32 else 1e-6)
    elif file.endswith("DNNConv2DForwardTest.cpp") and fn == "checkConv2DForward":
        p = _ints(f["helper_calls"][0]["args"])  # C H W Hf Wf sh sw ph pw
        inp, flt = M(args[0]), M(args[1])
        bias = np.zeros((1, 1), dt)
        res, oh, ow = backend.conv2d(inp, flt, bias, inp.shape[0], *p)
        _eq(res, M(args[2]))
    elif file.endswith("CUDA/DNNConvolutionTest.cpp") and fn == "direct":
        p = _ints(f["helper_calls"][0]["args"])
        inp, flt = M("input"), M("filter")
        res, oh, ow = backend.conv2d(inp, flt, None, inp.shape[0], *p)
        _eq(res, M("result"))
    elif "Pooling" in file and fn == "checkPoolingForward":
        if file.startswith("CUDA/"):
            raise Skip("CUDA/DNNPoolingTest.cpp is not part of the reference's test build and its expectation "
                       "belongs to other parameters than its call")
        p = _ints(f["helper_calls"][0]["args"])  # C H W ph pw sh sw padh padw
        inp = M(args[0])
        if "AVG" in c["name"]:
            res, oh, ow = backend.avgpool(inp, inp.shape[0], *p)
        else:
            res, oh, ow = backend.maxpool(inp, inp.shape[0], *p)
        _eq(res, M(args[1]))
    elif fn in ("checkBiasAddForward", "checkBiasAdd"):
        _eq(backend.bias_add(M(args[0]), M(args[1])), M(args[2]))
    elif "BatchNorm" in file and ("Inference" in fn or (fn == "direct" and "BatchNorm::Forward" in c["name"])):
        x = M("input")
        got = backend.batchnorm(x, M("gamma"), M("beta"), M("ema_mean"), M("ema_var"), 1e-5)
        _approx(got, M("result"), 1e-4)  # the reference compares with Approx().epsilon(1e-5) on ~unit values
    elif "Softmax" in file and fn == "direct":
        got = backend.softmax(M("input"))
        _approx(got, M("result"), 1e-6 if (dt == np.float32 or file.startswith("CUDA/")) else 1e-12)
    elif file.endswith("CUDA/DNNAffineTest.cpp") and fn == "direct":
        _eq(backend.affine(M("input"), M("weights"), M("bias")), M("result"))
    elif file.endswith("CUDA/DNNActivationTest.cpp") and fn == "direct":
        _eq(backend.relu(M("input")), M("result"))
        # ReLU == ewBinaryObjSca(MAX, x, 0): the reference has no CPU activation kernel
        _eq(backend.ew_binary_sca(BIN["MAX"], M("input"), 0.0), M("result"))
    elif fn == "checkTranspose":
        _eq(backend.transpose(M(args[0])), M(args[1]))
    elif file.endswith("ColBindTest.cpp") and fn == "direct" and "Frame" not in c["name"]:
        _eq(backend.col_bind(M("m0"), M("m1")), M("exp"))
    elif file.endswith("ExtractColTest.cpp") and fn in ("checkExtractCol", "checkExtractColThrow"):
        if "DenseMatrix" not in c["name"] and "arg" not in mats:
            raise Skip("frames are outside the dense float/double kernel set")
        arg = M(args[1])
        if not any(d["pos"] < pos for d in c["matrices"].get(args[2].strip(), [])):
            raise Skip("empty selection built without a literal")
        sel = matrix(mats[args[2].strip()], np.float64).astype(np.int64)
        if fn == "checkExtractColThrow":
            try:
                backend.extract_col(arg, sel)
            except OutOfRange:
                return
            raise AssertionError("expected std::out_of_range")
        exp = matrix(mats[args[3].strip()], dt)
        if exp.size == 0:
            exp = exp.reshape(arg.shape[0], 0)
        _eq(backend.extract_col(arg, sel), exp)
    elif fn == "checkConv2DBackwardData":
        # DNNConv2DBackwardTest.cpp:23-27: apply(filter, in, 2, 2, 1, 1, 1, 3, 3, 3, 2, 3, 2, 2, res)
        _eq(backend.conv2d_backward_data(M(args[1]), M(args[0]), 1, 3, 3, 3, 2, 2, 2, 2, 2, 1, 1), M(args[2]))
    elif fn == "checkConv2DBackwardFilter":
        # :53-57: apply(res, input, dOutput, 2, 2, 1, 1, 1, 3, 3, 3, 2, 3, 2, 2)
        _eq(backend.conv2d_backward_filter(M(args[0]), M(args[1]), 1, 3, 3, 3, 2, 2, 2, 2, 2, 1, 1), M(args[2]))
    elif fn in ("check_avg", "check_max") and file.endswith("DNNPoolingBackwardTest.cpp"):
        # DNNPoolingBackwardTest.cpp:41-51: apply(res, in, dOut, 2, 3, 3, 3, 2, 2, 2, 2, 1, 1)
        x, dout = matrix(mats["genInput"], dt), matrix(mats["genDOut"], dt)
        f = backend.avgpool_backward if fn == "check_avg" else backend.maxpool_backward
        _eq(f(x, dout, 2, 3, 3, 3, 2, 2, 2, 2, 1, 1), M(args[2]))
    elif fn == "checkBatchNorm2DBackward":
        # DNNBatchNorm2DBackwardTest.cpp:22-36; invVar is written there as 1 / sqrt(1.25f + 1e-5f)
        x, dout, gamma, mean = M(args[0]), M(args[1]), M(args[2]), M(args[3])
        inv_var = np.full(mean.shape, 1 / np.sqrt(np.float32(1.25) + np.float32(1e-5)), dtype=dt)
        dX, dG, dB = backend.batchnorm_backward(mean, inv_var, x, dout, gamma, 1e-5)
        _approx(dX, M(args[5]), 1e-5)
        _approx(dG.reshape(-1, 1), M(args[6]).reshape(-1, 1), 1e-4)
        _approx(dB.reshape(-1, 1), M(args[7]).reshape(-1, 1), 1e-5)
    elif fn == "checkBatchNorm2DTrainForward":
        # DNNBatchNorm2DForwardTest.cpp:51-64: epsilon 1e-5, mu 1
        x = M(args[0])
        res, nm, nv, mean, inv_var = backend.batchnorm_train_forward(x, M(args[1]), M(args[2]), M(args[3]), M(args[4]), 1e-5, 1.0)
        _approx(res, M(args[5]), 1e-4)
        # with mu = 1 the new moving averages are the batch statistics themselves
        C = mean.size
        per_c = x.reshape(x.shape[0], C, -1).transpose(1, 0, 2).reshape(C, -1).astype(np.float64)
        _approx(nm.reshape(-1, 1), per_c.mean(axis=1).reshape(-1, 1).astype(dt), 1e-5)
        _approx(nv.reshape(-1, 1), per_c.var(axis=1).reshape(-1, 1).astype(dt), 1e-4)
    else:
        raise Skip(f"{fn} is outside the dense float/double kernel set")
