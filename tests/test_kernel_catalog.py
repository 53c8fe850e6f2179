"""CPU: the generator of the HIP kernel library's entry points and catalog.

The names a DAPHNE program links against are fixed by the reference's generator
(src/runtime/local/kernels/genKernelInst.py:169-206). The reference tree holds a handful of such names as
literals - in its tests, its documentation and in the two compiler passes that spell a callee by hand - and
those pin the naming rule here: the generator is run on the kernel templates in question (api CPP, whose prefix
is a bare underscore) and must produce exactly those strings. The HIP names are the same rule with `HIP_`.
The catalog is checked against what src/parser/catalog/KernelCatalogParser.cpp:33-143 accepts.
"""
import importlib.util
import json
import re
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HIP_DIR = ROOT / "daphne_amd" / "cpp" / "src" / "runtime" / "local" / "kernels" / "HIP"
SPEC = HIP_DIR / "HIPkernels.json"


def load_generator():
    spec = importlib.util.spec_from_file_location("genHIPKernelInst", HIP_DIR / "genHIPKernelInst.py")
    mod = importlib.util.module_from_spec(spec)
    sys.modules["genHIPKernelInst"] = mod
    spec.loader.exec_module(mod)
    return mod


gen = load_generator()
DM = lambda vt: ["DenseMatrix", vt]  # noqa: E731


def template(header, op, tparams, rparams, ret="void", **kw):
    return {"header": header, "opName": op, "returnType": ret, "templateParams": [{"name": n} for n in tparams],
            "runtimeParams": [{"type": t, "name": n} for t, n in rparams], **kw}


EW_BINARY_MAT = template("EwBinaryMat.h", "ewBinaryMat", ["DTRes", "DTLhs", "DTRhs"],
                         [("BinaryOpCode", "opCode"), ("DTRes *&", "res"), ("const DTLhs *", "lhs"), ("const DTRhs *", "rhs")])
AGG_ALL = template("AggAll.h", "aggAll", ["VTRes", "DTArg"], [("AggOpCode", "opCode"), ("const DTArg *", "arg")], ret="VTRes")


def names(tmpl, values, op_codes, api="CPP"):
    return [w.func_name for w in gen.instantiate(tmpl, values, op_codes, api)]


def test_names_the_reference_holds_as_literals():
    # test/api/cli/extensibility/hint_kernel_success_4.daphne:3, hint_kernel_success_5.daphne:3
    got = names(EW_BINARY_MAT, [DM("int64_t")] * 3, ["ADD", "MUL"])
    assert got == ["_ewAdd__DenseMatrix_int64_t__DenseMatrix_int64_t__DenseMatrix_int64_t",
                   "_ewMul__DenseMatrix_int64_t__DenseMatrix_int64_t__DenseMatrix_int64_t"]
    # test/api/cli/extensibility/HintTest.cpp:66, hint_kernel_success_2.daphne:3: a scalar result comes first
    assert names(AGG_ALL, ["int64_t", DM("int64_t")], ["SUM"]) == ["_sumAll__int64_t__DenseMatrix_int64_t"]
    # doc/RunningDaphneLocally.md:140: scalar kernel, suffix Sca dropped
    sca = template("EwBinarySca.h", "ewBinarySca", ["TRes", "TLhs", "TRhs"],
                   [("BinaryOpCode", "opCode"), ("TLhs", "lhs"), ("TRhs", "rhs")], ret="TRes")
    assert names(sca, ["int32_t"] * 3, ["ADD"]) == ["_ewAdd__int32_t__int32_t__int32_t"]
    # test/api/cli/extensibility/HintTest.cpp:67: two results, then the arguments
    recode = template("Recode.h", "recode", ["DTRes", "DTDict", "DTArg"],
                      [("DTRes *&", "res"), ("DTDict *&", "dict"), ("const DTArg *", "arg"), ("bool", "orderPreserving")])
    assert names(recode, [DM("int64_t"), DM("double"), DM("double")], None) == [
        "_recode__DenseMatrix_int64_t__DenseMatrix_double__DenseMatrix_double__bool"]
    # src/compiler/lowering/RewriteToCallKernelOpPass.cpp:475-485: input arrays end in _variadic
    dist = template("DistributedPipeline.h", "distributedPipeline", ["DTRes"],
                    [("DTRes **", "outputs"), ("size_t", "numOutputs"), ("const Structure **", "inputs"), ("size_t", "numInputs"),
                     ("int64_t *", "outRows"), ("int64_t *", "outCols"), ("int64_t *", "splits"), ("int64_t *", "combines"),
                     ("const char *", "irCode")])
    assert names(dist, [DM("double")], None) == [
        "_distributedPipeline__DenseMatrix_double_variadic__size_t__Structure_variadic__size_t__int64_t__int64_t__int64_t"
        "__int64_t__char"]
    # src/compiler/lowering/LowerToLLVMPass.cpp:735-849, spelled piece by piece there
    vect = next(k["kernelTemplate"] for k in json.loads(SPEC.read_text()) if k["kernelTemplate"]["opName"] == "vectorizedPipeline")
    assert names(vect, [DM("double")], None) == [
        "_vectorizedPipeline__DenseMatrix_double_variadic__size_t__bool__Structure_variadic__size_t__int64_t__int64_t"
        "__int64_t__int64_t__size_t__void_variadic"]


def wrappers():
    return gen.generate(json.loads(SPEC.read_text()), "HIP")


def test_hip_names_follow_the_same_rule():
    by_name = {w.func_name: w for w in wrappers()}
    for expected in [
        "HIP_createHIPContext",
        "HIP_ewAdd__DenseMatrix_float__DenseMatrix_float__DenseMatrix_float",
        "HIP_ewBitwise_and__DenseMatrix_int64_t__DenseMatrix_int64_t__int64_t",
        "HIP_ewSqrt__DenseMatrix_double__DenseMatrix_double",
        "HIP_sumAll__double__DenseMatrix_double",
        "HIP_stddevCol__DenseMatrix_float__DenseMatrix_float",
        "HIP_idxminRow__DenseMatrix_size_t__DenseMatrix_float",
        "HIP_matMul__DenseMatrix_float__DenseMatrix_float__DenseMatrix_float__bool__bool",
        "HIP_syrk__DenseMatrix_double__DenseMatrix_double__bool",
        "HIP_fill__DenseMatrix_uint64_t__uint64_t__size_t__size_t",
        "HIP_extractCol__DenseMatrix_float__DenseMatrix_float__DenseMatrix_int64_t",
        "HIP_NN_Max_Forward__DenseMatrix_float__size_t__size_t__DenseMatrix_float" + "__size_t" * 10,
        "HIP_NN_Avg_Forward__DenseMatrix_double__size_t__size_t__DenseMatrix_double" + "__size_t" * 10,
        "HIP_NN_Relu_Forward__DenseMatrix_float__DenseMatrix_float",
        "HIP_NN_Affine_Forward__DenseMatrix_float__DenseMatrix_float__DenseMatrix_float__DenseMatrix_float",
        "HIP_Convolution_Forward__DenseMatrix_float__size_t__size_t__DenseMatrix_float__DenseMatrix_float__DenseMatrix_float"
        + "__size_t" * 10,
        "HIP_BatchNormInferenceForward__DenseMatrix_double" * 1 + "__DenseMatrix_double" * 5 + "__double",
        "HIP_Softmax__DenseMatrix_float__DenseMatrix_float",
        "HIP_BiasAdd__DenseMatrix_float__DenseMatrix_float__DenseMatrix_float",
        "HIP_vectorizedPipeline__DenseMatrix_float_variadic__size_t__bool__Structure_variadic__size_t__int64_t__int64_t"
        "__int64_t__int64_t__size_t__void_variadic",
    ]:
        assert expected in by_name, expected
    assert len(by_name) == len(wrappers()), "a function is generated twice"
    # the op code is a run-time argument of the kernel, or its first template argument for the NN kernels
    assert by_name["HIP_sumAll__double__DenseMatrix_double"].call == \
        "*res = HIP::aggAll<double, DenseMatrix<double>>(AggOpCode::SUM, arg, ctx)"
    assert by_name["HIP_NN_Relu_Forward__DenseMatrix_float__DenseMatrix_float"].call == \
        "HIP::NN::Activation::Forward<HIP::NN::Activation::ReLU, DenseMatrix<float>, DenseMatrix<float>>::apply(*res, data, ctx)"
    assert by_name["HIP_createHIPContext"].signature() == "void HIP_createHIPContext(int kId, DCTX(ctx))"


def test_every_device_kernel_of_the_reference_has_a_hip_entry():
    """The op mnemonics of the reference's CUDA catalog (kernels.json entries with api CUDA), minus the two value
    types the HIP library does not instantiate for fill (uint8_t, bool)."""
    mnemonics = {w.mnemonic for w in wrappers()}
    binary = "Add Sub Mul Div Pow Log Mod Eq Neq Lt Le Gt Ge Min Max And Or".split()
    expected = {f"ew{b}" for b in binary} | {"ewBitwise_and"}
    expected |= {f"{a}{dim}" for a in ("sum", "min", "max") for dim in ("All", "Row", "Col")}
    expected |= {"colBind", "extractCol", "fill", "matMul", "transpose", "solve", "syrk", "gemv", "NN_Avg_Forward",
                 "NN_Max_Forward", "NN_Relu_Forward", "NN_Affine_Forward", "BatchNormInferenceForward", "Convolution_Forward",
                 "Softmax", "BiasAdd", "createHIPContext"}
    assert expected <= mnemonics, sorted(expected - mnemonics)
    # beyond the reference's device set: unary operators, moments, positions of extrema, the training kernels
    assert {"ewSqrt", "ewIsnan", "meanAll", "varCol", "stddevRow", "idxminRow", "idxmaxCol", "conv2DBackwardData",
            "conv2DBackwardFilter", "maxPoolBackward", "avgPoolBackward", "batchNorm2DTrainForward", "batchNorm2DBackward",
            "vectorizedPipeline"} <= mnemonics


# What KernelCatalogParser.cpp:33-97 puts into its type map: CompilerUtils::mlirTypeToCppTypeName of every scalar
# type, of DenseMatrix / CSRMatrix / list / column / memref over it, and Structure, Frame, DaphneContext.
SCALARS = ["double", "float", "int64_t", "int32_t", "int8_t", "uint64_t", "uint32_t", "uint8_t", "bool", "size_t", "std::string"]
KNOWN_TYPES = set(SCALARS) | {f"{c}<{s}>" for s in SCALARS for c in ("DenseMatrix", "CSRMatrix", "Column")} | \
    {"Structure", "Frame", "DaphneContext"}


def test_catalog_is_what_the_catalog_parser_reads(tmp_path):
    out_cpp, out_cat = tmp_path / "k.cpp", tmp_path / "lib" / "HIPcatalog.json"
    subprocess.run([sys.executable, str(HIP_DIR / "genHIPKernelInst.py"), str(SPEC), str(out_cpp), str(out_cat), "HIP"], check=True)
    catalog = json.loads(out_cat.read_text())
    assert isinstance(catalog, list) and len(catalog) == len(wrappers())
    cpp = out_cpp.read_text()
    for rec in catalog:
        assert set(rec) == {"opMnemonic", "kernelFuncName", "resTypes", "argTypes", "backend", "libPath"}
        assert rec["backend"] == "HIP" and rec["libPath"] == "libHIPKernels.so"
        assert re.fullmatch(r"HIP_[A-Za-z0-9_]+", rec["kernelFuncName"])
        assert f"void {rec['kernelFuncName']}(" in cpp
        if rec["opMnemonic"] in ("vectorizedPipeline",):
            continue  # called by a hand-spelled name, not looked up by types (LowerToLLVMPass.cpp:735-849)
        for t in rec["resTypes"] + rec["argTypes"]:
            assert t in KNOWN_TYPES, (rec["kernelFuncName"], t)
    one = next(r for r in catalog if r["kernelFuncName"] == "HIP_matMul__DenseMatrix_float__DenseMatrix_float__DenseMatrix_float__bool__bool")
    assert one == {"opMnemonic": "matMul", "kernelFuncName": one["kernelFuncName"], "resTypes": ["DenseMatrix<float>"],
                   "argTypes": ["DenseMatrix<float>", "DenseMatrix<float>", "bool", "bool"], "backend": "HIP",
                   "libPath": "libHIPKernels.so"}
    agg = next(r for r in catalog if r["kernelFuncName"] == "HIP_sumAll__float__DenseMatrix_float")
    assert agg["resTypes"] == ["float"] and agg["argTypes"] == ["DenseMatrix<float>"]
    # every entry point has the instrumented body: timing hooks and the call-site error (genKernelInst.py:236-262)
    assert cpp.count("preKernelInstrumentation(kId, ctx);") == len(catalog)
    assert cpp.count("throw ErrorHandler::runtimeError(kId, e.what(), &(ctx->dispatchMapping));") == len(catalog)


def test_built_library_exports_every_catalog_entry():
    from daphne_amd import build as b

    if not (b.KERNEL_LIB_PATH.exists() and b.KERNEL_CATALOG_PATH.exists()):
        b.build_kernel_library(verbose=False)
    out = subprocess.run(["nm", "-D", "--defined-only", str(b.KERNEL_LIB_PATH)], capture_output=True, text=True, check=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if line.strip()}
    catalog = json.loads(b.KERNEL_CATALOG_PATH.read_text())
    assert [r["kernelFuncName"] for r in catalog] == [w.func_name for w in wrappers()], "the built catalog is stale"
    missing = [r["kernelFuncName"] for r in catalog if r["kernelFuncName"] not in exported]
    assert not missing, missing[:5]


def test_instantiation_with_wrong_arity_is_refused():
    with pytest.raises(ValueError, match="template parameters"):
        gen.instantiate(EW_BINARY_MAT, [DM("float")], ["ADD"], "HIP")
