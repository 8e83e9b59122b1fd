// Added to the Honeycrisp target of the Linux package: `autoreleasepool` is an Objective-C
// runtime facility that Foundation only provides on Apple platforms; the reference calls it
// around worker-thread jobs and data-loading loops (Sources/Honeycrisp/Backend.swift:151,
// DataUtil.swift:15,61,106). Without Objective-C there is nothing to drain.
#if !canImport(ObjectiveC)
  @inline(__always)
  public func autoreleasepool<Result>(invoking body: () throws -> Result) rethrows -> Result {
    try body()
  }
#endif
