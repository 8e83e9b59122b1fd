"""swift/honeycrisp-linux/preexpand_macros.py: the ahead-of-time expansion of Honeycrisp's two
macros (Sources/HCBacktrace/Macros/RecordCaller.swift:8-170, AlwaysAssert.swift:5-20), checked on
synthetic Swift snippets against what the macro implementations generate, and as whole-tree
properties on an upstream checkout when one is present."""
import os
import re
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "swift", "honeycrisp-linux"))
import preexpand_macros as pm  # noqa: E402

EXTRA = "function: StaticString = #function, file: StaticString = #filePath, line: UInt = #line"
RECORD_TAIL = ", function: function, file: file, line: line)"


def squeeze(text):
    return re.sub(r"\s+", " ", text).strip()


def test_always_assert_forms():
    assert pm.expand("#alwaysAssert(x > 0)") == "(!(x > 0) ? alwaysAssert(false, nil) : ())"
    assert pm.expand('#alwaysAssert(a == b, "differ")') == '(!(a == b) ? alwaysAssert(false, "differ") : ())'
    # the literal false short-cuts the condition (AlwaysAssert.swift:16-18)
    assert pm.expand('{ _ in #alwaysAssert(false, "twice") }') == '{ _ in alwaysAssert(false, "twice") }'
    with pytest.raises(pm.MacroError):
        pm.expand("#alwaysAssert(a, b, c)")


def test_always_assert_arguments_with_commas_brackets_and_interpolations():
    src = '''#alwaysAssert(
      axis == nil || f(axis!, [1, 2]) < shape.count,
      "axis \\(axis!) out of bounds for shape \\(shape), e.g. \\(g(1, "x)")))"
    )'''
    out = pm.expand(src)
    assert out.startswith("(!(axis == nil || f(axis!, [1, 2]) < shape.count) ? alwaysAssert(false, \"axis \\(axis!)")
    assert out.endswith(') : ())') and '\\(g(1, "x)"))' in out
    # generic arguments hold commas too
    assert pm.expand("#alwaysAssert(Dictionary<String, Int>().isEmpty, m)") == \
        "(!(Dictionary<String, Int>().isEmpty) ? alwaysAssert(false, m) : ())"
    # nested: the inner one is expanded too
    out = pm.expand("#alwaysAssert(check { #alwaysAssert(y) }, m)")
    assert "#alwaysAssert" not in out and out.count("alwaysAssert(false") == 2


def test_macro_names_in_comments_and_strings_are_left_alone():
    src = '''/// Use `@recordCaller` and #alwaysAssert(x) like this.
/* block #alwaysAssert(a) /* nested @recordCaller */ still comment */
let s = "#alwaysAssert(q) @recordCaller }"
let m = """
  #alwaysAssert(in a multi-line string)
  """
let r = #"raw "quoted" #alwaysAssert(r)"#
'''
    assert pm.expand(src) == src


def test_record_caller_plain_method():
    src = '''class Foo {
  @recordCaller
  private func _printNumbers(x: Int) {
    for i in 0..<x { print(i) }
  }
}
'''
    out = pm.expand(src)
    assert "@recordCaller" not in out
    assert "  private func _printNumbers(x: Int) {\n    for i in 0..<x { print(i) }\n  }\n" in out    # original kept
    assert squeeze("public func printNumbers(x: Int, %s) { Backtrace.record({ _printNumbers(x: x) }%s }" % (EXTRA, RECORD_TAIL)) \
        in squeeze(out)


def test_record_caller_effects_labels_inout_generics():
    src = '''extension Tensor {
  @recordCaller
  private func _copyToArray<T: TensorElement>(_ out: inout [T]) async throws {
    try await fill(&out)
  }

  @recordCaller
  private static func _withGrad<T>(enabled flag: Bool, _ fn: () async throws -> T) async rethrows
    -> T
  {
    try await run(flag, fn)
  }

  @recordCaller
  internal func _positiveAxis(_ axis: Int?) -> Int? { axis }

  @recordCaller
  static private func _make(shape: [Int] = [1, 2], dtype: DType = .float32, fn: @escaping @Sendable (Tensor) -> Void) -> Tensor {
    Tensor()
  }

  @recordCaller
  private func _callAsFunction() -> Tensor { self }
}
'''
    out = squeeze(pm.expand(src))
    assert "@recordCaller" not in out
    # async + throws: await inside try, around both the record call and the inner call; inout passed with &
    assert squeeze("public func copyToArray<T: TensorElement>(_ out: inout [T], %s) async throws { "
                   "try await Backtrace.record({ try await _copyToArray(&out) }%s }" % (EXTRA, RECORD_TAIL)) in out
    # rethrows counts as throwing; the multi-line signature tail is kept; external label passed, `_` not
    assert squeeze("public static func withGrad<T>(enabled flag: Bool, _ fn: () async throws -> T, %s) async rethrows -> T { "
                   "try await Backtrace.record({ try await _withGrad(enabled: flag, fn) }%s }" % (EXTRA, RECORD_TAIL)) in out
    # `throws` inside a parameter's closure type does not make the function throwing; internal stays internal
    assert squeeze("internal func positiveAxis(_ axis: Int?, %s) -> Int? { Backtrace.record({ _positiveAxis(axis) }%s }"
                   % (EXTRA, RECORD_TAIL)) in out
    # defaults with commas and attributed closure types survive; modifiers in either order
    assert squeeze("static public func make(shape: [Int] = [1, 2], dtype: DType = .float32, fn: @escaping @Sendable (Tensor) -> Void, "
                   "%s) -> Tensor { Backtrace.record({ _make(shape: shape, dtype: dtype, fn: fn) }%s }" % (EXTRA, RECORD_TAIL)) in out
    # no parameters: no leading comma
    assert squeeze("public func callAsFunction(%s) -> Tensor { Backtrace.record({ _callAsFunction() }%s }"
                   % (EXTRA, RECORD_TAIL)) in out


def test_record_caller_keeps_bodies_with_asserts_and_braces_in_strings():
    src = '''struct S {
  @recordCaller
  private func _check(_ n: Int) throws -> String {
    #alwaysAssert(n >= 0, "negative: \\(n) }")
    return "}{"
  }
}
'''
    out = pm.expand(src)
    assert '(!(n >= 0) ? alwaysAssert(false, "negative: \\(n) }") : ())' in out
    assert squeeze("public func check(_ n: Int, %s) throws -> String { try Backtrace.record({ try _check(n) }%s }"
                   % (EXTRA, RECORD_TAIL)) in squeeze(out)
    assert pm.match_bracket(out, out.index("{")) == out.rindex("}")    # braces in strings do not count


def test_record_caller_rejects_what_the_macro_rejects():
    with pytest.raises(pm.MacroError):
        pm.expand("@recordCaller\nvar x = 1\n")


@pytest.mark.skipif(not os.path.isdir("/root/reference/Sources"), reason="no upstream checkout here")
def test_whole_upstream_tree_expands_cleanly(tmp_path):
    """Every macro use in code is gone afterwards, every attribute produced exactly one generated
    function whose name is the original's without the underscore, braces stay balanced, and files
    without macros come out byte for byte."""
    src = "/root/reference/Sources"
    n = pm.expand_tree(src, str(tmp_path))
    assert n >= 40
    attributes = asserts = generated = 0
    for root, _dirs, files in os.walk(src):
        for f in files:
            if not f.endswith(".swift"):
                continue
            path = os.path.join(root, f)
            before = open(path).read()
            after = open(os.path.join(str(tmp_path), os.path.relpath(path, src))).read()
            a, b = len(pm.code_positions(before, pm.ATTRIBUTE)), len(pm.code_positions(before, pm.ASSERT))
            attributes, asserts = attributes + a, asserts + b
            if a == 0 and b == 0:
                assert after == before
                continue
            assert not pm.code_positions(after, pm.ATTRIBUTE) and not pm.code_positions(after, pm.ASSERT)
            generated += after.count("Backtrace.record({ ") - before.count("Backtrace.record({ ")
            assert after.count(EXTRA) - before.count(EXTRA) == a
            depth, i = 0, 0
            while i < len(after):
                j = pm.skip_trivia_or_string(after, i)
                if j is not None:
                    i = j
                    continue
                depth += {"{": 1, "}": -1}.get(after[i], 0)
                i += 1
            assert depth == 0, path
            for m in re.finditer(r"Backtrace\.record\(\{ (?:try )?(?:await )?(_\w+)\(", after):
                assert re.search(r"func %s\b" % re.escape(m.group(1)[1:]), after), m.group(1)
    assert attributes == generated and attributes > 100 and asserts > 200
