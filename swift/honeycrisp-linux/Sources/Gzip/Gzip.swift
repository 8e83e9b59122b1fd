// Stand-in for the GzipSwift package (a network dependency of the reference, Package.swift:28).
// HCTestUtils imports it for one fixture, the gzipped conv2d test vectors
// (Sources/HCTestUtils/BackendTests.swift:1850-1854); everything else in the test suite is
// independent of it. `gunzipped()` therefore only has to exist: it throws, which fails that one
// convolution test (convolutions are not on this backend's path) and leaves the rest running.
import Foundation

public struct GzipError: Error, CustomStringConvertible {
  public let description = "gzip decompression is not available in the offline Linux build"
}

extension Data {
  public func gunzipped() throws -> Data {
    throw GzipError()
  }
}
