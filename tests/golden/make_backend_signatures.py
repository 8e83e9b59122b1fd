"""Writes tests/golden/backend_swift_signatures.json: the `open func` declarations of the reference's
Backend class (Sources/Honeycrisp/Backend.swift:170-892) as data (name, generic parameters,
argument labels, parameter types, effects, result type, where clause, line), which
tests/test_swift_signatures.py compares the overrides of swift/Sources/HoneycrispHIP/HIPBackend.swift
with. Run from the repository root where the reference checkout is present:
    python tests/golden/make_backend_signatures.py /root/reference
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from swift_signatures import functions  # noqa: E402


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    src = open(os.path.join(ref, "Sources", "Honeycrisp", "Backend.swift")).read()
    decls = functions(src, "open")
    with open(os.path.join(HERE, "backend_swift_signatures.json"), "w") as f:
        json.dump({"source": "Sources/Honeycrisp/Backend.swift", "open_funcs": decls}, f, indent=1)
    print(len(decls), "declarations")


if __name__ == "__main__":
    main()
