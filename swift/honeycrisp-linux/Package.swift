// swift-tools-version: 5.10
// Offline Linux package of Honeycrisp, for use next to the MI355X backend (../Package.swift
// refers to it by path). The Honeycrisp sources themselves are not part of this directory:
// `prepare.py <honeycrisp checkout>` copies them into Derived/ byte for byte except for the
// expansion of the two macros (preexpand_macros.py), so that neither swift-syntax nor any other
// network dependency of the upstream manifest (Package.swift:25-30 there) is needed:
//
//   upstream                                   here
//   HCBacktraceMacros (swift-syntax)           expanded ahead of time; Interface/Macros.swift dropped
//   import Accelerate                          Sources/Accelerate: C target with the symbols in use
//   import Metal / MetalPerformanceShaders*    empty modules; BackendMPS.swift left out
//   CoreMLBuilder, BackendCoreML.swift         left out
//   Gzip (HCTestUtils)                         Sources/Gzip stand-in
//   autoreleasepool                            Sources/LinuxCompat/Autoreleasepool.swift, copied into Honeycrisp
//
// Not built in the authoring environment or on the GPU machines used for testing (no Swift
// toolchain on either); the C target and the macro expansion are tested from Python.
import PackageDescription

let package = Package(
  name: "Honeycrisp",
  products: [
    .library(name: "HCBacktrace", targets: ["HCBacktrace"]),
    .library(name: "Honeycrisp", targets: ["Honeycrisp"]),
    .library(name: "HCTestUtils", targets: ["HCTestUtils"]),
  ],
  targets: [
    .target(
      name: "Accelerate", path: "Sources/Accelerate",
      cSettings: [.unsafeFlags(["-ffp-contract=off", "-fno-fast-math"])],
      linkerSettings: [.linkedLibrary("dl"), .linkedLibrary("m"), .linkedLibrary("pthread")]),
    .target(name: "Metal", path: "Sources/Metal"),
    .target(name: "MetalPerformanceShaders", path: "Sources/MetalPerformanceShaders"),
    .target(name: "MetalPerformanceShadersGraph", path: "Sources/MetalPerformanceShadersGraph"),
    .target(name: "Gzip", path: "Sources/Gzip"),
    .target(name: "HCBacktrace", path: "Derived/HCBacktrace/Interface"),
    .target(
      name: "Honeycrisp",
      dependencies: [
        "HCBacktrace", "Accelerate", "Metal", "MetalPerformanceShaders", "MetalPerformanceShadersGraph",
      ],
      path: "Derived/Honeycrisp",
      exclude: ["Honeycrisp.docc"]),
    .target(
      name: "HCTestUtils", dependencies: ["Honeycrisp", "Gzip"], path: "Derived/HCTestUtils",
      resources: [.process("Resources")]),
  ]
)
