"""A small reader of Swift method declarations: enough of the grammar to list the `func`s of a
class with their argument labels, parameter types, generic parameters, `where` clause and result
type. It serves the one check this environment can give the Swift layer (no Swift compiler here or
on the GPU machines): that every `override` in HIPBackend.swift names a method the reference's
`Backend` really declares, with the same labels and types."""
import re


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _balanced(text, start, open_ch, close_ch):
    """Index just past the bracket that closes the one at text[start]."""
    depth = 0
    for i in range(start, len(text)):
        if text[i] == open_ch:
            depth += 1
        elif text[i] == close_ch:
            depth -= 1
            if depth == 0:
                return i + 1
    raise ValueError("unbalanced %s at %d" % (open_ch, start))


def _split_top_level(text, sep=",", angle=True):
    """Pieces of `text` between separators that sit outside every bracket. `angle` says whether
    < > count as brackets (they do in types, not in expressions: `a[..<n]`, `x < y`)."""
    opening, closing = ("([<{", ")]>}") if angle else ("([{", ")]}")
    parts, depth, cur = [], 0, ""
    for ch in text:
        if ch in opening:
            depth += 1
        elif ch in closing:
            depth -= 1
        if ch == sep and depth == 0:
            parts.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        parts.append(cur)
    return parts


def _squeeze(text):
    return re.sub(r"\s+", " ", text).strip()


def _parameter(text):
    """('label', 'Type') of one parameter; the label is '_' for an unlabelled one."""
    text = _squeeze(text)
    names, typ = text.split(":", 1)
    typ = _squeeze(_split_top_level(typ, "=")[0])          # a default value is not part of the signature
    names = names.split()
    return (names[0], typ)


def functions(text, modifiers):
    """Every `<modifiers> func` of `text` as a dict: name, generics, labels, types, result, where."""
    text = _strip_comments(text)
    out = []
    for m in re.finditer(r"\b%s\s+func\s+([A-Za-z_][A-Za-z0-9_]*)" % r"\s+".join(map(re.escape, modifiers.split())), text):
        pos = m.end()
        generics = ""
        while text[pos].isspace():
            pos += 1
        if text[pos] == "<":
            end = _balanced(text, pos, "<", ">")
            generics = _squeeze(text[pos + 1:end - 1])
            pos = end
        while text[pos].isspace():
            pos += 1
        end = _balanced(text, pos, "(", ")")
        params = [_parameter(p) for p in _split_top_level(text[pos + 1:end - 1]) if p.strip()]
        tail = text[end:text.index("{", end)]
        effects = _squeeze(tail.split("->")[0])
        result, where = "", ""
        if "->" in tail:
            rest = tail.split("->", 1)[1]
            bits = re.split(r"\bwhere\b", rest, maxsplit=1)
            result = _squeeze(bits[0])
            where = _squeeze(bits[1]) if len(bits) > 1 else ""
        out.append({"name": m.group(1), "generics": generics, "labels": [p[0] for p in params],
                    "types": [p[1] for p in params], "effects": effects, "result": result, "where": where,
                    "line": text.count("\n", 0, m.start()) + 1})
    return out


def key(f):
    return (f["name"], f["generics"], tuple(f["labels"]), tuple(f["types"]), f["effects"], f["result"], f["where"])


def called_symbols(text, prefix="hc_"):
    """Identifiers starting with `prefix` that the text calls (name followed by an opening parenthesis)."""
    return sorted(set(re.findall(r"\b(%s[a-z0-9_]+)\s*\(" % re.escape(prefix), _strip_comments(text))))
