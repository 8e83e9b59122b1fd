#!/usr/bin/env python3
"""Derives the Linux source tree of Honeycrisp from an upstream checkout.

    prepare.py <honeycrisp checkout> [<output dir, default: Derived/ next to this file>]

Copies Sources/HCBacktrace/Interface, Sources/Honeycrisp and Sources/HCTestUtils, expanding the two macros in every Swift file (preexpand_macros.py) and
changing nothing else, and leaves out what cannot exist off Apple platforms or needs the network:

  Sources/HCBacktrace/Macros/            the macro implementations (swift-syntax)
  Sources/HCBacktrace/Interface/Macros.swift   the macro declarations (expanded ahead of time instead)
  Sources/Honeycrisp/BackendMPS.swift, BackendCoreML.swift, Resources/kernels.txt   Metal / CoreML backends
  Tests/HoneycrispTests/                 instantiates MPSBackend and CoreMLBackend; the backend package's own
                                         test target runs the same shared BackendTests under CPUBackend and HIPBackend

and adds Sources/LinuxCompat/Autoreleasepool.swift to the Honeycrisp target. Package.swift in
this directory builds the result; ../Package.swift (the MI355X backend) depends on it by path.
"""
import os
import shutil
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import preexpand_macros  # noqa: E402

LEFT_OUT = {
    os.path.join("HCBacktrace", "Interface", "Macros.swift"),
    os.path.join("Honeycrisp", "BackendMPS.swift"),
    os.path.join("Honeycrisp", "BackendCoreML.swift"),
    os.path.join("Honeycrisp", "Resources", "kernels.txt"),
}


def derive(checkout, out):
    copied, expanded = 0, 0
    pairs = [(os.path.join(checkout, "Sources", "HCBacktrace", "Interface"), os.path.join(out, "HCBacktrace", "Interface")),
             (os.path.join(checkout, "Sources", "Honeycrisp"), os.path.join(out, "Honeycrisp")),
             (os.path.join(checkout, "Sources", "HCTestUtils"), os.path.join(out, "HCTestUtils"))]
    for src, dst in pairs:
        for root, _dirs, files in os.walk(src):
            for name in files:
                path = os.path.join(root, name)
                if os.path.relpath(path, os.path.join(checkout, "Sources")) in LEFT_OUT:
                    continue
                target = os.path.join(dst, os.path.relpath(path, src))
                os.makedirs(os.path.dirname(target), exist_ok=True)
                if name.endswith(".swift"):
                    with open(path) as fh:
                        text = fh.read()
                    new = preexpand_macros.expand(text)
                    expanded += new != text
                    with open(target, "w") as fh:
                        fh.write(new)
                else:
                    shutil.copyfile(path, target)
                copied += 1
    shutil.copyfile(os.path.join(HERE, "Sources", "LinuxCompat", "Autoreleasepool.swift"),
                    os.path.join(out, "Honeycrisp", "Autoreleasepool.swift"))
    return copied, expanded


def main(argv):
    if len(argv) not in (2, 3):
        sys.stderr.write(__doc__)
        return 2
    out = argv[2] if len(argv) == 3 else os.path.join(HERE, "Derived")
    copied, expanded = derive(argv[1], out)
    print("wrote %d files to %s (%d with macros expanded)" % (copied, out, expanded))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
