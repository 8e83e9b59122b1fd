// Runs the reference's shared backend suite (HCTestUtils.BackendTests) with HIPBackend as the
// default backend, the way HoneycrispTests.runInBackends does for CPU and MPS
// (Tests/HoneycrispTests/HoneycrispTests.swift:9-38).
import HCTestUtils
import Honeycrisp
import HoneycrispHIP
import XCTest

final class HIPBackendTests: XCTestCase {
  func runInHIP(_ fn: () async throws -> Void) async throws {
    let saved = Backend.defaultBackend
    Backend.defaultBackend = try HIPBackend()
    defer { Backend.defaultBackend = saved }
    try await fn()
  }

  func testCast() async throws { try await runInHIP(BackendTests.testCast) }
  func testAdd() async throws { try await runInHIP(BackendTests.testAdd) }
  func testSub() async throws { try await runInHIP(BackendTests.testSub) }
  func testMul() async throws { try await runInHIP(BackendTests.testMul) }
  func testDiv() async throws { try await runInHIP(BackendTests.testDiv) }
  func testMod() async throws { try await runInHIP(BackendTests.testMod) }
  func testFusedAddMul() async throws { try await runInHIP(BackendTests.testFusedAddMul) }
  func testFusedNormalize() async throws { try await runInHIP(BackendTests.testFusedNormalize) }
  func testSum() async throws { try await runInHIP(BackendTests.testSum) }
  func testGather() async throws { try await runInHIP(BackendTests.testGather) }
  func testMatrixMatrixProduct() async throws { try await runInHIP(BackendTests.testMatrixMatrixProduct) }
  func testBatchedMatmul() async throws { try await runInHIP(BackendTests.testBatchedMatmul) }
  func testMatrixVectorProduct() async throws { try await runInHIP(BackendTests.testMatrixVectorProduct) }
  func testIndexing() async throws { try await runInHIP(BackendTests.testIndexing) }
  func testElemwise() async throws { try await runInHIP(BackendTests.testElemwise) }
  func testMinMax() async throws { try await runInHIP(BackendTests.testMinMax) }
  func testExpandAndRepeat() async throws { try await runInHIP(BackendTests.testExpandAndRepeat) }
  func testBinaryBroadcast() async throws { try await runInHIP(BackendTests.testBinaryBroadcast) }
  func testFusedBroadcast() async throws { try await runInHIP(BackendTests.testFusedBroadcast) }
  func testSoftmax() async throws { try await runInHIP(BackendTests.testSoftmax) }
  func testCreateFromData() async throws { try await runInHIP(BackendTests.testCreateFromData) }
  func testEquals() async throws { try await runInHIP(BackendTests.testEquals) }
  func testComparison() async throws { try await runInHIP(BackendTests.testComparison) }
  func testBitwise() async throws { try await runInHIP(BackendTests.testBitwise) }
  func testProd() async throws { try await runInHIP(BackendTests.testProd) }
  func testCumulativeSum() async throws { try await runInHIP(BackendTests.testCumulativeSum) }
  func testCumulativeProd() async throws { try await runInHIP(BackendTests.testCumulativeProd) }
  func testArgsort() async throws { try await runInHIP(BackendTests.testArgsort) }
  func testRepeat() async throws { try await runInHIP(BackendTests.testRepeat) }
  func testTriangular() async throws { try await runInHIP(BackendTests.testTriangular) }
  func testChunk() async throws { try await runInHIP(BackendTests.testChunk) }
  func testClamp() async throws { try await runInHIP(BackendTests.testClamp) }
  func testAllSome() async throws { try await runInHIP(BackendTests.testAllSome) }
  func testConcatInner() async throws { try await runInHIP(BackendTests.testConcatInner) }
  func testConcatOuter() async throws { try await runInHIP(BackendTests.testConcatOuter) }
  func testWhen() async throws { try await runInHIP(BackendTests.testWhen) }
  func testOneHot() async throws { try await runInHIP(BackendTests.testOneHot) }
  func testAdam() async throws { try await runInHIP(BackendTests.testAdam) }
  func testMulGrad() async throws { try await runInHIP(BackendTests.testMulGrad) }
  func testMSEGrad() async throws { try await runInHIP(BackendTests.testMSEGrad) }
}
