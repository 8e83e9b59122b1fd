#!/usr/bin/env python3
"""Source-to-source expansion of Honeycrisp's two macros, so that the package builds without the
swift-syntax dependency (which SwiftPM fetches from the network, Package.swift:25-37).

  @recordCaller   (peer macro, Sources/HCBacktrace/Macros/RecordCaller.swift:8-170)
      Attached to `private func _name(params) [async] [throws] -> R { body }`. The macro adds a second
      function next to it: the name without its leading underscore, `private` turned into
      `public`, the parameters followed by
          function: StaticString = #function, file: StaticString = #filePath, line: UInt = #line
      and a body that calls the original inside `Backtrace.record({ ... }, function:file:line:)`,
      with `await` / `try` where the original is `async` / `throws` (or `rethrows`). A parameter
      whose first name is `_` is passed without a label, an `inout` parameter with `&`.
      Here: the attribute is removed and that second function is written out after the original.

  #alwaysAssert(condition[, message])   (expression macro, Macros/AlwaysAssert.swift:5-20)
      -> `(!(condition) ? alwaysAssert(false, message) : ())`, or `alwaysAssert(false, message)`
      when the condition is the literal `false`; a missing message is `nil`.

Comments and string literals (with interpolations, multi-line and raw forms) are skipped, so a
macro name inside a doc comment or a string is left alone.

Usage: preexpand_macros.py <in.swift> [<out.swift>]     one file (stdout by default)
       preexpand_macros.py --tree <src_dir> <dst_dir>   every .swift file under src_dir
"""
import os
import re
import sys

ATTRIBUTE = "@recordCaller"
ASSERT = "#alwaysAssert"
OPEN = {"(": ")", "[": "]", "{": "}"}


class MacroError(Exception):
    pass


def skip_string(text, i):
    """`i` is at the opening quote (after any `#`s of a raw string, whose count is `hashes`).
    Returns the index after the closing delimiter."""
    hashes = 0
    j = i
    while j > 0 and text[j - 1] == "#":
        hashes += 1
        j -= 1
    multi = text.startswith('"""', i)
    quote = '"""' if multi else '"'
    close = quote + "#" * hashes
    escape = "\\" + "#" * hashes
    i += len(quote)
    n = len(text)
    while i < n:
        if text.startswith(escape, i):
            k = i + len(escape)
            if k < n and text[k] == "(":      # interpolation: ordinary code up to the matching ")"
                i = match_bracket(text, k) + 1
            else:
                i = k + 1
            continue
        if text.startswith(close, i):
            return i + len(close)
        if not multi and text[i] == "\n":
            raise MacroError("unterminated string literal")
        i += 1
    raise MacroError("unterminated string literal")


def skip_trivia_or_string(text, i):
    """If a comment or a string literal starts at `i`, the index after it; else None."""
    if text.startswith("//", i):
        j = text.find("\n", i)
        return len(text) if j < 0 else j
    if text.startswith("/*", i):      # block comments nest in Swift
        depth, i = 1, i + 2
        while depth and i < len(text):
            if text.startswith("/*", i):
                depth, i = depth + 1, i + 2
            elif text.startswith("*/", i):
                depth, i = depth - 1, i + 2
            else:
                i += 1
        return i
    if text[i] == '"':
        return skip_string(text, i)
    return None


def match_bracket(text, i):
    """Index of the bracket that closes the one at `i`."""
    stack = [OPEN[text[i]]]
    i += 1
    n = len(text)
    while i < n:
        j = skip_trivia_or_string(text, i)
        if j is not None:
            i = j
            continue
        c = text[i]
        if c in OPEN:
            stack.append(OPEN[c])
        elif c in ")]}":
            if c != stack.pop():
                raise MacroError("mismatched bracket at offset %d" % i)
            if not stack:
                return i
        i += 1
    raise MacroError("unclosed bracket")


def split_top_level(text, sep=","):
    """Split at separators that are outside brackets, generic argument lists, strings and comments."""
    parts, start, i, angle = [], 0, 0, 0
    n = len(text)
    while i < n:
        j = skip_trivia_or_string(text, i)
        if j is not None:
            i = j
            continue
        c = text[i]
        if c in OPEN:
            i = match_bracket(text, i) + 1
            continue
        if text.startswith("->", i):
            i += 2
            continue
        # `<` opens a generic argument list only where Swift itself reads it so: directly after a
        # name (`Dictionary<String, Int>`); with a space in front it is the comparison operator
        if c == "<" and i > 0 and (text[i - 1].isalnum() or text[i - 1] == "_") and i + 1 < n and not text[i + 1].isspace():
            angle += 1
        elif c == ">" and angle:
            angle -= 1
        elif c == sep and angle == 0:
            parts.append(text[start:i])
            start = i + 1
        i += 1
    parts.append(text[start:])
    return parts


def find_top_level(text, token):
    """Offset of the first `token` outside brackets, strings and comments, or -1."""
    i, n = 0, len(text)
    while i < n:
        j = skip_trivia_or_string(text, i)
        if j is not None:
            i = j
            continue
        if text.startswith(token, i):
            return i
        if text[i] in OPEN:
            i = match_bracket(text, i) + 1
            continue
        i += 1
    return -1


def code_positions(text, token):
    """Offsets of `token` in code (not inside comments or strings), as a whole word."""
    out, i, n = [], 0, len(text)
    while i < n:
        j = skip_trivia_or_string(text, i)
        if j is not None:
            i = j
            continue
        if text.startswith(token, i):
            end = i + len(token)
            if end >= n or not (text[end].isalnum() or text[end] == "_"):
                out.append(i)
            i = end
            continue
        i += 1
    return out


def expand_always_assert(text):
    """Replace every #alwaysAssert(...) in code, innermost first (arguments may hold another one)."""
    while True:
        positions = code_positions(text, ASSERT)
        if not positions:
            return text
        i = positions[-1]       # the last one holds no other: replacing it never invalidates the rest
        j = i + len(ASSERT)
        while text[j].isspace():
            j += 1
        if text[j] != "(":
            raise MacroError("#alwaysAssert without an argument list")
        close = match_bracket(text, j)
        args = [a.strip() for a in split_top_level(text[j + 1:close])]
        if args and args[-1] == "":     # trailing comma
            args.pop()
        if len(args) not in (1, 2):
            raise MacroError("alwaysAssert expects 1 or 2 arguments, but got %d" % len(args))
        condition = args[0]
        message = args[1] if len(args) == 2 else "nil"
        if condition == "false":
            new = "alwaysAssert(false, %s)" % message
        else:
            new = "(!(%s) ? alwaysAssert(false, %s) : ())" % (condition, message)
        text = text[:i] + new + text[close + 1:]


IDENT = r"[A-Za-z_][A-Za-z0-9_]*|`[^`]+`"


def parse_parameter(param):
    """(label or None, argument name, is_inout) of one parameter of a declaration."""
    names, rest = None, None
    depth_parts = split_top_level(param, ":")
    if len(depth_parts) < 2:
        raise MacroError("cannot parse parameter %r" % param)
    head, rest = depth_parts[0], ":".join(depth_parts[1:])
    # drop attributes in front of the names (rare)
    head = re.sub(r"@\w+(\([^)]*\))?\s*", "", head).strip()
    names = re.findall(IDENT, head)
    if not names or len(names) > 2:
        raise MacroError("cannot parse parameter names in %r" % param)
    first, second = names[0], (names[1] if len(names) == 2 else None)
    type_part = split_top_level(rest, "=")[0]
    is_inout = re.search(r"(^|[\s(])inout\s", " " + type_part) is not None
    return (None if first == "_" else first), (second or first), is_inout


def expand_record_caller(text):
    """Remove each @recordCaller attribute and append the function the macro would generate."""
    while True:
        positions = code_positions(text, ATTRIBUTE)
        if not positions:
            return text
        at = positions[-1]      # back to front: earlier offsets stay valid
        line_start = text.rfind("\n", 0, at) + 1
        indent = text[line_start:at]
        if indent.strip():
            raise MacroError("@recordCaller must stand at the start of a line")
        i = at + len(ATTRIBUTE)
        # declaration head: modifiers and attributes up to `func`
        m = re.compile(r"\s*((?:(?:@\w+(?:\([^)]*\))?|[a-z]+(?:\((?:set)\))?)\s+)*?)func\s+(" + IDENT + r")").match(text, i)
        if not m:
            raise MacroError("@recordCaller only works on functions")
        modifiers, name = m.group(1), m.group(2)
        decl_start = m.start(1) if m.group(1) else text.index("func", m.start())
        j = m.end()
        generics = ""
        while text[j].isspace():
            j += 1
        if text[j] == "<":
            depth, k = 0, j
            while True:
                if text.startswith("->", k):
                    k += 2
                    continue
                if text[k] == "<":
                    depth += 1
                elif text[k] == ">":
                    depth -= 1
                    if depth == 0:
                        break
                k += 1
            generics = text[j:k + 1]
            j = k + 1
            while text[j].isspace():
                j += 1
        if text[j] != "(":
            raise MacroError("no parameter list after func %s" % name)
        params_close = match_bracket(text, j)
        params_text = text[j + 1:params_close]
        # the rest of the signature runs up to the body's opening brace
        k = params_close + 1
        while True:
            t = skip_trivia_or_string(text, k)
            if t is not None:
                k = t
                continue
            if text[k] == "{":
                break
            if text[k] in "([":
                k = match_bracket(text, k) + 1
                continue
            k += 1
        tail = text[params_close + 1:k]
        body_close = match_bracket(text, k)
        arrow = find_top_level(tail, "->")
        effects = tail if arrow < 0 else tail[:arrow]     # before the return arrow
        effects = re.split(r"\bwhere\b", effects)[0]
        is_async = re.search(r"\basync\b", effects) is not None
        is_throws = re.search(r"\b(re)?throws\b", effects) is not None

        params = [p for p in (q.strip() for q in split_top_level(params_text)) if p]
        call_args = []
        for p in params:
            label, arg, is_inout = parse_parameter(p)
            expr = ("&" if is_inout else "") + arg
            call_args.append(expr if label is None else "%s: %s" % (label, expr))
        new_name = name[name.index("_") + 1:] if "_" in name else name
        prefix = ("try " if is_throws else "") + ("await " if is_async else "")
        inner = "%s%s(%s)" % (prefix, name, ", ".join(call_args))
        extra = "function: StaticString = #function, file: StaticString = #filePath, line: UInt = #line"
        new_params = (params_text.rstrip().rstrip(",") + ", " if params else "") + extra
        new_modifiers = re.sub(r"\bprivate\b", "public", modifiers)
        peer = ("\n\n%s%sfunc %s%s(%s)%s{\n%s  %sBacktrace.record({ %s }, function: function, file: file, line: line)\n%s}"
                % (indent, new_modifiers, new_name, generics, new_params, tail if tail.strip() else " ",
                   indent, prefix, inner, indent))
        # original without the attribute (and its line), then the generated function
        text = text[:line_start] + indent + text[decl_start:body_close + 1] + peer + text[body_close + 1:]


def expand(text):
    return expand_record_caller(expand_always_assert(text))


def expand_tree(src, dst):
    count = 0
    for root, _dirs, files in os.walk(src):
        for f in files:
            if not f.endswith(".swift"):
                continue
            path = os.path.join(root, f)
            out = os.path.join(dst, os.path.relpath(path, src))
            os.makedirs(os.path.dirname(out), exist_ok=True)
            with open(path) as fh:
                text = fh.read()
            try:
                new = expand(text)
            except MacroError as e:
                raise MacroError("%s: %s" % (path, e))
            with open(out, "w") as fh:
                fh.write(new)
            count += 1
    return count


def main(argv):
    if len(argv) == 4 and argv[1] == "--tree":
        print("expanded %d files" % expand_tree(argv[2], argv[3]))
        return 0
    if len(argv) in (2, 3) and not argv[1].startswith("-"):
        with open(argv[1]) as fh:
            new = expand(fh.read())
        if len(argv) == 3:
            with open(argv[2], "w") as fh:
                fh.write(new)
        else:
            sys.stdout.write(new)
        return 0
    sys.stderr.write(__doc__)
    return 2


if __name__ == "__main__":
    sys.exit(main(sys.argv))
