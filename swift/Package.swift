// swift-tools-version: 5.10
// SwiftPM package of the MI355X backend for Honeycrisp. NOT built in the authoring environment
// (no Swift toolchain there); it is the binding a maintainer adds next to Honeycrisp.
//
// CHCHIP is the thin C target: it only re-exports include/hchip.h and links libhchip.so,
// which wraps hipMalloc / hipMemcpyAsync / hipModuleLaunchKernel over the embedded gfx950
// code objects. Build libhchip.so first: `python -m honeycrisp_amd.csrc.build`.
import PackageDescription

let package = Package(
  name: "HoneycrispHIP",
  products: [
    .library(name: "HoneycrispHIP", targets: ["HoneycrispHIP"]),
    .executable(name: "HCMatrixBench", targets: ["HCMatrixBench"]),
  ],
  dependencies: [
    // The offline Linux package of Honeycrisp: honeycrisp-linux/prepare.py derives its sources from an
    // upstream checkout (macros expanded ahead of time; Accelerate, Metal and Gzip stand-ins in place).
    .package(path: "honeycrisp-linux")
  ],
  targets: [
    .systemLibrary(name: "CHCHIP", path: "Sources/CHCHIP"),
    .target(
      name: "HoneycrispHIP",
      dependencies: ["CHCHIP", .product(name: "Honeycrisp", package: "honeycrisp-linux")],
      linkerSettings: [
        .unsafeFlags(["-L../honeycrisp_amd/csrc", "-Xlinker", "-rpath", "-Xlinker", "../honeycrisp_amd/csrc"])
      ]),
    .executableTarget(
      name: "HCMatrixBench",
      dependencies: ["HoneycrispHIP", .product(name: "Honeycrisp", package: "honeycrisp-linux")]),
    .testTarget(
      name: "HoneycrispHIPTests",
      dependencies: [
        "HoneycrispHIP", .product(name: "Honeycrisp", package: "honeycrisp-linux"),
        .product(name: "HCTestUtils", package: "honeycrisp-linux"),
      ]),
  ]
)
