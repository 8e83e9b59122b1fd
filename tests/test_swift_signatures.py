"""The Swift layer (swift/Sources) has never met a Swift compiler: there is none in this image or on
the GPU machines. What can be checked without one is checked here, as text: every `override open
func` of HIPBackend.swift must name a method that the reference's `Backend` declares `open`, with
the same generic parameters, argument labels, parameter types, effects, result type and `where`
clause (Sources/Honeycrisp/Backend.swift:170-892, kept as data in
tests/golden/backend_swift_signatures.json); and every hc_* function the Swift sources call must be
declared in include/hchip.h and be called with as many arguments as its prototype takes."""
import json
import os
import re

import pytest

from swift_signatures import _balanced, _split_top_level, _strip_comments, called_symbols, functions, key

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SWIFT = os.path.join(ROOT, "swift", "Sources")
GOLDEN = os.path.join(ROOT, "tests", "golden", "backend_swift_signatures.json")
REFERENCE = "/root/reference/Sources/Honeycrisp/Backend.swift"


def reference_decls():
    return json.load(open(GOLDEN))["open_funcs"]


def swift_sources():
    for folder, _, files in os.walk(SWIFT):
        for name in sorted(files):
            if name.endswith(".swift"):
                yield os.path.join(folder, name)


def header_prototypes():
    """name -> number of parameters, for every function include/hchip.h declares."""
    text = _strip_comments(open(os.path.join(ROOT, "include", "hchip.h")).read())
    protos = {}
    for m in re.finditer(r"\b(hc_[a-z0-9_]+)\s*\(", text):
        end = _balanced(text, m.end() - 1, "(", ")")
        if not text[end:].lstrip().startswith(";"):
            continue
        args = text[m.end():end - 1].strip()
        protos[m.group(1)] = 0 if args in ("", "void") else len(_split_top_level(args))
    return protos


def test_the_parser_on_a_declaration_it_must_get_right():
    text = '''
    open class B {
      /// doc
      override open func pow<T: NumericTensorElement>(
        _ a: Tensor.Data, _ b: T, scale: T, scales: Tensor.Data?, count: Int = 3, dtype: Tensor.DType
      ) async throws -> Tensor.Data where T: Foo { body() }
      open func plain() { }
    }'''
    (f,) = functions(text, "override open")
    assert f["name"] == "pow" and f["generics"] == "T: NumericTensorElement"
    assert f["labels"] == ["_", "_", "scale", "scales", "count", "dtype"]
    assert f["types"] == ["Tensor.Data", "T", "T", "Tensor.Data?", "Int", "Tensor.DType"]
    assert f["effects"] == "async throws" and f["result"] == "Tensor.Data" and f["where"] == "T: Foo"
    assert [g["name"] for g in functions(text, "open")] == ["pow", "plain"]


def test_golden_signatures_are_those_of_the_reference_checkout():
    if not os.path.exists(REFERENCE):
        pytest.skip("no reference checkout on this machine: the committed signatures stand")
    now = functions(open(REFERENCE).read(), "open")
    assert [key(f) for f in now] == [key(f) for f in reference_decls()]
    names = {f["name"] for f in now}
    for hot in ("matmul", "batchedMatmul", "binaryOp", "elemwise", "pow", "reduce", "gather", "axisPermutation"):
        assert hot in names


def test_every_override_matches_a_declaration_of_the_reference_backend():
    declared = {key(f) for f in reference_decls()}
    path = os.path.join(SWIFT, "HoneycrispHIP", "HIPBackend.swift")
    ours = functions(open(path).read(), "override open")
    assert len(ours) >= 30
    wrong = []
    for f in ours:
        if key(f) not in declared:
            near = [r for r in reference_decls() if r["name"] == f["name"]]
            wrong.append("HIPBackend.swift:%d %s%s: no such declaration in Backend.swift (same name there: %s)" % (
                f["line"], f["name"], tuple(f["labels"]), [(r["line"], r["labels"], r["types"]) for r in near]))
    assert not wrong, "\n".join(wrong)
    # the hot path of the build is among them
    ours_names = {f["name"] for f in ours}
    for hot in ("matmul", "batchedMatmul", "binaryOp", "elemwise", "pow", "reduce", "gather", "axisPermutation",
                "logSoftmax", "cast", "mulAdd", "addMul", "constant", "compare", "when", "triangular"):
        assert hot in ours_names, hot
    # all three binaryOp and compare forms (tensor-tensor, tensor-scalar, scalar-tensor)
    assert sum(f["name"] == "binaryOp" for f in ours) == 3 and sum(f["name"] == "compare" for f in ours) == 3


def test_every_library_call_of_the_swift_sources_is_declared_with_that_many_arguments():
    protos = header_prototypes()
    assert "hc_matmul" in protos and protos["hc_matmul"] == 12
    types = {"hc_strides", "hc_device_info"}           # structs of the header, constructed by name
    problems = []
    for path in swift_sources():
        text = _strip_comments(open(path).read())
        for name in called_symbols(text):
            if name in types:
                continue
            if name not in protos:
                problems.append("%s calls %s, which include/hchip.h does not declare" % (os.path.relpath(path, ROOT), name))
                continue
            for m in re.finditer(r"\b%s\s*\(" % re.escape(name), text):
                end = _balanced(text, m.end() - 1, "(", ")")
                args = text[m.end():end - 1].strip()
                n = 0 if not args else len(_split_top_level(args, angle=False))
                if n != protos[name]:
                    line = text.count("\n", 0, m.start()) + 1
                    problems.append("%s:%d %s called with %d arguments, declared with %d" % (
                        os.path.relpath(path, ROOT), line, name, n, protos[name]))
    assert not problems, "\n".join(problems)
