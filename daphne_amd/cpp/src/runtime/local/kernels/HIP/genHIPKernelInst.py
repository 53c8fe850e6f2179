#!/usr/bin/env python3
"""Generates the pre-compiled HIP kernel library's entry points and its kernel catalog.

    python3 genHIPKernelInst.py HIPkernels.json OUT.cpp OUT_catalog.json [API]

DAPHNE's compiled programs reach a kernel through a plain C function per (kernel, op code, types), found by
name in a catalog that is read at start-up. This script writes both for the HIP backend from a specification in
the format of DAPHNE's src/runtime/local/kernels/kernels.json:

  * OUT.cpp: one `extern "C" void HIP_<mnemonic>__<types>(results..., arguments..., int kId, DaphneContext *ctx)`
    per instantiation, which times the call when statistics are on and turns any exception into the run-time
    error of the call site the dispatch id stands for;
  * OUT_catalog.json: one record per function (`opMnemonic`, `kernelFuncName`, `resTypes`, `argTypes`,
    `backend`, `libPath`), the fields src/parser/catalog/KernelCatalogParser.cpp:117-143 reads.

Names, parameter lists and catalog records follow the rules of the reference's generator
(src/runtime/local/kernels/genKernelInst.py:132-284) so that a specification entry with api "HIP" yields the
same function as its "CUDA" entry does there, with the prefix `HIP_` and the namespace `HIP::`:

  mnemonic   the kernel name without trailing Sca / Mat / Obj, `::` as `_`; with an op code, the op-code family
             (the op-code type without `OpCode` and without namespaces, e.g. `Binary`, `Agg`, `Pooling`) is
             replaced inside it by the op code (`ewBinaryMat` + ADD -> `ewAdd`, `aggAll` + SUM -> `sumAll`,
             `NN::Pooling::Forward` + MAX -> `NN_Max_Forward`);
  types      every parameter's C++ type, in order, a scalar result first: namespaces, `const`, pointer and
             reference signs dropped, `<` `,` and blanks as `_`; an input array (`T **`, or marked variadic) ends
             in `_variadic`; joined by `__`.

The script has no dependencies beyond the standard library and can be imported: `generate(spec, api)` returns
the wrappers as objects, which the tests use to call the built library by catalog.
"""
from __future__ import annotations

import json
import re
import sys
from dataclasses import dataclass, field
from pathlib import Path

# kernels whose call sites carry no dispatch id (genKernelInst.py:156-166)
_UNINSTRUMENTED = ("map", "createDaphneContext", "destroyDaphneContext")
# a catalog record's argument types end before the first of these (genKernelInst.py:268-273)
_ARG_TYPES_STOP = ("void", "mlir::daphne::GroupEnum", "CompareOperation")

_TEMPLATE_ARG_NS = re.compile(r"^(.*)<.*::(.*)>(.*)$")
_OUTER_NS = re.compile(r"^.*::(.*)$")


def cpp_type(value) -> str:
    """["DenseMatrix", "float"] -> DenseMatrix<float>; a plain string is a type already."""
    if isinstance(value, str):
        return value
    if len(value) == 2:
        return f"{value[0]}<{value[1]}>"
    if len(value) == 3:
        return f"{value[0]}<{value[1]}<{value[2]}>>"
    raise ValueError(f"template value nested too deep: {value!r}")


def without_namespaces(t: str) -> str:
    """`const DenseMatrix<std::string> *` -> `const DenseMatrix<string> *`, `mlir::daphne::GroupEnum` -> `GroupEnum`."""
    t = _TEMPLATE_ARG_NS.sub(r"\1<\2>\3", t)
    return _OUTER_NS.sub(r"\1", t)


@dataclass
class Param:
    type: str
    name: str
    is_output: bool = False
    is_variadic: bool = False

    def name_part(self) -> str:
        t = without_namespaces(self.type).replace("const ", "")
        t = t.replace(" **", "" if self.is_output else "_variadic")
        t = t.replace(" *", "_variadic" if self.is_variadic else "")
        for old, new in (("& ", ""), ("<", "_"), (">", ""), (",", "_"), (" ", "_")):
            t = t.replace(old, new)
        return t

    def catalog_type(self) -> str:
        return self.type.replace(" **", "").replace(" *", "").replace("const ", "")

    def call_argument(self) -> str:
        return ("*" if self.is_output and self.type.endswith("**") else "") + self.name


@dataclass
class Wrapper:
    """One generated entry point."""
    op_name: str           # the kernel template, e.g. NN::Pooling::Forward
    mnemonic: str          # e.g. NN_Max_Forward
    func_name: str         # e.g. HIP_NN_Max_Forward__DenseMatrix_float__size_t__...
    params: list[Param]    # the C parameters before kId and ctx
    op_code: str | None
    has_kid: bool
    has_ctx: bool
    call: str              # the C++ expression the body evaluates
    header: str
    api: str
    template_values: list = field(default_factory=list)

    def signature(self) -> str:
        ps = [f"{p.type} {p.name}" for p in self.params]
        if self.has_kid:
            ps.append("int kId")
        if self.has_ctx:
            ps.append("DCTX(ctx)")
        return f"void {self.func_name}({', '.join(ps)})"

    def definition(self) -> str:
        if not self.has_kid:
            return f"    {self.signature()} {{\n        {self.call};\n    }}\n"
        return (f"    {self.signature()} {{\n"
                f"        try {{\n"
                f"            preKernelInstrumentation(kId, ctx);\n"
                f"            {self.call};\n"
                f"            postKernelInstrumentation(kId, ctx);\n"
                f"        }} catch (std::exception &e) {{\n"
                f"            throw ErrorHandler::runtimeError(kId, e.what(), &(ctx->dispatchMapping));\n"
                f"        }}\n"
                f"    }}\n")

    def catalog_record(self) -> dict:
        args = []
        for p in self.params:
            if p.is_output:
                continue
            t = p.catalog_type()
            if t in _ARG_TYPES_STOP:
                break
            args.append(t)
        return {
            "opMnemonic": self.mnemonic,
            "kernelFuncName": self.func_name,
            "resTypes": [p.catalog_type() for p in self.params if p.is_output],
            "argTypes": args,
            "backend": self.api,
            # the catalog file is stored next to the kernel libraries
            "libPath": "libAllKernels.so" if self.api == "CPP" else f"lib{self.api}Kernels.so",
        }


def op_code_family(op_code_type: str) -> str:
    """`BinaryOpCode` -> `Binary`, `NN::PoolingOpCode` -> `Pooling`."""
    word = op_code_type[: -len("OpCode")]
    return word.split("::")[-1]


def mnemonic_of(op_name: str, op_code_type: str | None, op_code: str | None) -> str:
    name = op_name
    while name[-3:] in ("Sca", "Mat", "Obj"):
        name = name[:-3]
    name = name.replace("::", "_")
    if op_code is not None:
        family = op_code_family(op_code_type)
        name = name.replace(family, op_code[0].upper() + op_code[1:].lower())
        name = name.replace(family.lower(), op_code.lower())
    return name


def _bind_params(template: dict, values: list, with_op_code: bool) -> list[Param]:
    tparams = template["templateParams"]
    if len(tparams) != len(values):
        raise ValueError(f'kernel "{template["opName"]}" has {len(tparams)} template parameters, '
                         f"but an instantiation supplies {len(values)}")
    runtime = template["runtimeParams"][1:] if with_op_code else template["runtimeParams"]
    params: list[Param] = []
    if template["returnType"] != "void":
        params.append(Param(f'{template["returnType"]} *', "res", is_output=True))
    for rp in runtime:
        params.append(Param(rp["type"], rp["name"], is_output=bool(rp.get("isOutput") or rp.get("isReturnValue")),
                            is_variadic=bool(rp.get("isVariadic"))))
    for p in params:
        for tp, tv in zip(tparams, values):
            if not isinstance(tv, str):
                p.type = p.type.replace(f'typename {tp["name"]}::VT', tv[1])
            p.type = p.type.replace(tp["name"], cpp_type(tv))
        if p.type.endswith("*&"):          # a data object the kernel may create: passed as T **
            p.type = p.type[:-2] + "**"
            p.is_output = True
        elif p.type.endswith("&"):         # a scalar result by reference: the reference passes it by value
            p.type = p.type[:-1]
            p.is_output = True
    return params


def instantiate(template: dict, values: list, op_codes: list[str] | None, api: str) -> list[Wrapper]:
    op_name = template["opName"]
    op_code_type = template["runtimeParams"][0]["type"] if op_codes is not None else None
    as_template_param = template.get("opCodeAsTemplateParam") == 1
    params = _bind_params(template, values, op_codes is not None)
    types_for_name = "__".join(p.name_part() for p in params)
    if types_for_name:
        types_for_name = "__" + types_for_name
    has_ctx = op_name != "createDaphneContext"
    has_kid = op_name not in _UNINSTRUMENTED and "distributed" not in op_name
    scope = "" if api == "CPP" else api + "::"
    prefix = "_" if api == "CPP" else api + "_"
    first_arg = 0 if template["returnType"] == "void" else 1

    out = []
    for op_code in (op_codes if op_codes is not None else [None]):
        mnemonic = mnemonic_of(op_name, op_code_type, op_code)
        targs = [cpp_type(v) for v in values]
        args = [p.call_argument() for p in params[first_arg:]]
        if op_code is not None:
            if as_template_param:
                targs.insert(0, f'{scope}{op_code_type[: -len("OpCode")]}::{op_code}')
            else:
                args.insert(0, f"{op_code_type}::{op_code}")
        if has_ctx:
            args.append("ctx")
        call = scope + op_name + (f'<{", ".join(targs)}>' if values else "")
        call += ("::apply(" if as_template_param else "(") + ", ".join(args) + ")"
        if template["returnType"] != "void":
            call = "*res = " + call
        out.append(Wrapper(op_name, mnemonic, prefix + mnemonic + types_for_name, [Param(**vars(p)) for p in params],
                           op_code, has_kid, has_ctx, call, template["header"], api, values))
    return out


def generate(spec: list, api: str = "HIP") -> list[Wrapper]:
    """All wrappers the specification asks for under `api`, in specification order."""
    wrappers: list[Wrapper] = []
    for kernel in spec:
        template = kernel["kernelTemplate"]
        if "api" in kernel:
            groups = [g for g in kernel["api"] if api in g["name"]]
        elif api == "CPP":
            groups = [kernel]
        else:
            groups = []
        for g in groups:
            for values in g["instantiations"]:
                wrappers.extend(instantiate(template, values, g.get("opCodes"), api))
    return wrappers


def render_cpp(wrappers: list[Wrapper], api: str = "HIP") -> str:
    headers = []
    for w in wrappers:
        h = f"#include <runtime/local/kernels/{w.header}>" if api == "CPP" else \
            f"#include <runtime/local/kernels/{api}/{w.header}>"
        if h not in headers:
            headers.append(h)
    lines = ["// Generated by genHIPKernelInst.py - do not edit.",
             "#include <stdexcept>",
             "#include <util/ErrorHandler.h>",
             "#include <runtime/local/context/DaphneContext.h>",
             "#include <runtime/local/instrumentation/KernelInstrumentation.h>",
             *headers, "", 'extern "C" {']
    last = None
    for w in wrappers:
        if w.op_name != last:
            lines += ["    // " + "-" * 76, "    // " + w.op_name, "    // " + "-" * 76]
            last = w.op_name
        lines.append(w.definition().rstrip("\n"))
    if any(w.op_name == "fusedPipeline" for w in wrappers):
        # not kernels (and not in the catalog): how the calling thread's last fusedPipeline call ran
        lines += ["    // " + "-" * 76,
                  "    // diagnostics of fusedPipeline: 1 one kernel per batch, 0 operator by operator (and why), -1 none yet",
                  "    // " + "-" * 76,
                  f"    int {api}_fusedPipeline_lastMode() {{ return {api}::fusedPipelineLastMode(); }}",
                  f"    const char *{api}_fusedPipeline_lastReason() {{ return {api}::fusedPipelineLastReason().c_str(); }}"]
    lines += ["}", ""]
    return "\n".join(lines)


def render_catalog(wrappers: list[Wrapper]) -> str:
    return json.dumps([w.catalog_record() for w in wrappers], indent=2) + "\n"


def main(argv: list[str]) -> int:
    if len(argv) not in (4, 5) or argv[1] in ("-h", "--help"):
        print(__doc__)
        return 0 if len(argv) > 1 and argv[1] in ("-h", "--help") else 1
    spec_path, cpp_path, catalog_path = map(Path, argv[1:4])
    api = argv[4] if len(argv) == 5 else "HIP"
    wrappers = generate(json.loads(spec_path.read_text()), api)
    names = [w.func_name for w in wrappers]
    if len(set(names)) != len(names):
        dup = sorted({n for n in names if names.count(n) > 1})
        raise SystemExit(f"the specification yields the same function more than once: {dup[:5]}")
    cpp_path.parent.mkdir(parents=True, exist_ok=True)
    catalog_path.parent.mkdir(parents=True, exist_ok=True)
    cpp_path.write_text(render_cpp(wrappers, api))
    catalog_path.write_text(render_catalog(wrappers))
    print(f"[genHIPKernelInst] {len(wrappers)} entry points -> {cpp_path}, catalog -> {catalog_path}")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
