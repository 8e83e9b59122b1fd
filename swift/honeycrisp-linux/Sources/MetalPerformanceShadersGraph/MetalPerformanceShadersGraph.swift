// Empty stand-in for Apple's MetalPerformanceShadersGraph framework on Linux. Honeycrisp imports the module in files
// that are kept in a Linux build (Sources/Honeycrisp/Broadcast.swift:2, BackendWrapper.swift:3-5)
// without using any of its symbols there; the only file that does use them, BackendMPS.swift, is
// left out of the Linux package.
