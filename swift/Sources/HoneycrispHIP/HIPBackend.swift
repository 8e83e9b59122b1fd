// HIPBackend: Honeycrisp `Backend` for one AMD Instinct MI355X (gfx950).
//
// `Backend.defaultBackend = try HIPBackend()` is the whole integration: Tensor, autodiff,
// Trainable and Linear are untouched. The class derives from CPUBackend (as MPSBackend does,
// BackendMPS.swift:10) so that every op it does not override, and the Philox random
// generator, keep working on the host; the overrides below enqueue one hchip call each on the
// context's in-order stream and return a device buffer (`HIPData`) immediately.
//
// Not compiled in the authoring environment, nor on the GPU machines it was tested on (neither
// has a Swift toolchain): written against Sources/Honeycrisp/Backend.swift:170-815 and the C ABI
// in include/hchip.h, unverified by a compiler.
import CHCHIP
import Foundation
import Honeycrisp

private func hcDType(_ dtype: Tensor.DType) -> Int32 {
  switch dtype {
  case .int64: Int32(HC_I64.rawValue)
  case .bool: Int32(HC_BOOL.rawValue)
  case .float16: Int32(HC_F16.rawValue)
  case .float32: Int32(HC_F32.rawValue)
  }
}

private func hcStrides(_ s: BroadcastStrides) -> hc_strides {
  precondition(s.shape.count <= Int(HC_MAX_DIMS), "at most \(HC_MAX_DIMS) axes are supported")
  var out = hc_strides()
  out.ndim = UInt32(s.shape.count)
  withUnsafeMutableBytes(of: &out.shape) { p in
    for (i, x) in s.shape.enumerated() { p.storeBytes(of: Int64(x), toByteOffset: i * 8, as: Int64.self) }
  }
  withUnsafeMutableBytes(of: &out.strides) { p in
    for (i, x) in s.strides.enumerated() { p.storeBytes(of: Int64(x), toByteOffset: i * 8, as: Int64.self) }
  }
  return out
}

open class HIPBackend: CPUBackend, @unchecked Sendable {

  /// Device buffer backing a tensor (Tensor.Data, Tensor.swift:69-85). Freed stream-ordered,
  /// so dropping the last reference right after a consumer was enqueued is safe.
  public final class HIPData: Tensor.Data, @unchecked Sendable {
    public let backend: HIPBackend
    public let pointer: UnsafeMutableRawPointer
    public let byteCount: Int
    /// Set by axisPermutation: what this index vector permutes (lets gather copy directly).
    public var permutation: (permutation: [Int], shape: [Int])? = nil

    init(backend: HIPBackend, byteCount: Int) throws {
      self.backend = backend
      self.byteCount = byteCount
      var p: UnsafeMutableRawPointer? = nil
      try backend.check(hc_malloc(backend.ctx, byteCount, &p), allocating: byteCount)
      self.pointer = p!
    }

    deinit { _ = hc_free(backend.ctx, pointer) }

    public func wait() async throws {
      try await backend.waitForStream()
    }

    public func onCPU<T>(_ fn: (_: UnsafeRawPointer) async throws -> T) async throws -> T {
      let host = UnsafeMutableRawPointer.allocate(byteCount: max(byteCount, 1), alignment: 16)
      defer { host.deallocate() }
      try await backend.waitForStream()  // do not block a cooperative thread on the copy
      try backend.check(hc_memcpy_d2h(backend.ctx, host, pointer, byteCount))
      return try await fn(host)
    }

    public func mutateOnCPU<T>(_ fn: (_: UnsafeMutableRawPointer) async throws -> T) async throws -> T {
      let host = UnsafeMutableRawPointer.allocate(byteCount: max(byteCount, 1), alignment: 16)
      defer { host.deallocate() }
      let result = try await fn(host)
      try backend.check(hc_memcpy_h2d(backend.ctx, pointer, host, byteCount))
      return result
    }
  }

  let ctx: OpaquePointer

  /// `batching` > 0: the library lists the launches of the backend calls and enqueues them in
  /// batches of at most that many, each batch rewritten (a Linear layer's bias, activation and
  /// residual go into the product's kernel, LayerNorm / softmax / attention become one kernel
  /// each) with the bits of the call-by-call result; anything that reads or waits for a result
  /// (`Tensor.Data.onCPU`, `wait()`) enqueues what is listed first, and so does a device that has
  /// run out of work once `idleAfter` launches are listed. `batching: 0` = one launch per call
  /// (what the C ABI does unless told otherwise).
  public init(device: Int = 0, batching: Int = 256, idleAfter: Int = 16) throws {
    var c: OpaquePointer? = nil
    let status = hc_init(Int32(device), &c)
    guard status == HC_OK.rawValue, let c = c else {
      throw BackendError.failedToLoadKernels(String(cString: hc_last_error_string()))
    }
    ctx = c
    super.init()
    try check(hc_set_batching(ctx, batching, idleAfter))
  }

  deinit { hc_shutdown(ctx) }

  /// hchip status -> BackendError (Backend.swift:6-16).
  func check(_ status: Int32, allocating bytes: Int = 0) throws {
    if status == HC_OK.rawValue { return }
    let msg = String(cString: hc_last_error_string())
    switch UInt32(status) {
    case HC_ERR_ALLOC.rawValue: throw BackendError.allocationFailed(bytes)
    case HC_ERR_LOAD.rawValue, HC_ERR_NO_DEVICE.rawValue: throw BackendError.failedToLoadKernels(msg)
    case HC_ERR_UNSUPPORTED.rawValue: throw BackendError.notImplemented(msg)
    default: throw BackendError.kernelFailed(msg)
    }
  }

  /// Resume once everything enqueued so far has completed, without blocking the calling
  /// cooperative thread (hipLaunchHostFunc resumes the continuation from a runtime thread;
  /// precedent: BackendMPS.swift:2663-2720).
  func waitForStream() async throws {
    final class Box { let c: CheckedContinuation<Void, Never>; init(_ c: CheckedContinuation<Void, Never>) { self.c = c } }
    var status: Int32 = 0
    await withCheckedContinuation { (c: CheckedContinuation<Void, Never>) in
      let box = Unmanaged.passRetained(Box(c))
      status = hc_launch_host_func(ctx, { raw in
        let box = Unmanaged<Box>.fromOpaque(raw!).takeRetainedValue()
        box.c.resume()
      }, box.toOpaque())
      if status != HC_OK.rawValue {
        box.release()
        c.resume()
      }
    }
    try check(status)
  }

  /// Device pointer for any Tensor.Data; foreign data (CPUData, another backend's) is uploaded
  /// (cf. MPSBackend.gpuBuffer, BackendMPS.swift:585-620). The returned HIPData keeps an
  /// uploaded copy alive until the op has been enqueued.
  func device(_ data: Tensor.Data) async throws -> HIPData {
    if let d = data as? HIPData, d.backend === self { return d }
    let out = try HIPData(backend: self, byteCount: data.byteCount)
    try await data.onCPU { host in
      try self.check(hc_memcpy_h2d(self.ctx, out.pointer, host, data.byteCount))
    }
    return out
  }

  func output(_ byteCount: Int) throws -> HIPData { try HIPData(backend: self, byteCount: byteCount) }

  // MARK: - hot path

  override open func matmul(
    a: Tensor.Data, transA: Bool, b: Tensor.Data, transB: Bool, transOut: Bool, rows: Int, inner: Int,
    cols: Int, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    try await batchedMatmul(
      matrixCount: 1, a: a, transA: transA, b: b, transB: transB, transOut: transOut, rows: rows,
      inner: inner, cols: cols, dtype: dtype)
  }

  override open func batchedMatmul(
    matrixCount: Int, a: Tensor.Data, transA: Bool, b: Tensor.Data, transB: Bool, transOut: Bool,
    rows: Int, inner: Int, cols: Int, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else {
      return try await super.batchedMatmul(
        matrixCount: matrixCount, a: a, transA: transA, b: b, transB: transB, transOut: transOut,
        rows: rows, inner: inner, cols: cols, dtype: dtype)
    }
    let (da, db) = (try await device(a), try await device(b))
    let out = try output(matrixCount * rows * cols * dtype.byteSize)
    try check(
      hc_matmul(
        ctx, hcDType(dtype), Int64(matrixCount), da.pointer, transA ? 1 : 0, db.pointer, transB ? 1 : 0,
        transOut ? 1 : 0, Int64(rows), Int64(inner), Int64(cols), out.pointer))
    return out
  }

  override open func binaryOp(
    _ a: BroadcastData, _ b: BroadcastData, op: NumericBinaryOp, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else { return try await super.binaryOp(a, b, op: op, dtype: dtype) }
    let (da, db) = (try await device(a.data), try await device(b.data))
    var (sa, sb) = (hcStrides(a.strides), hcStrides(b.strides))
    let out = try output(a.strides.shape.product() * dtype.byteSize)
    try check(hc_binary_op(ctx, hcOp(op), hcDType(dtype), da.pointer, &sa, db.pointer, &sb, out.pointer))
    return out
  }

  override open func binaryOp<T: NumericTensorElement>(
    _ a: Tensor.Data, _ b: T, op: NumericBinaryOp, count: Int, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else { return try await super.binaryOp(a, b, op: op, count: count, dtype: dtype) }
    let da = try await device(a)
    let out = try output(count * dtype.byteSize)
    try check(
      hc_binary_op_scalar(
        ctx, hcOp(op), hcDType(dtype), da.pointer, b.toFloat(), dtype == .int64 ? b.toInt64() : 0, 0,
        out.pointer, count))
    return out
  }

  override open func binaryOp<T: NumericTensorElement>(
    _ a: T, _ b: Tensor.Data, op: NumericBinaryOp, count: Int, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else { return try await super.binaryOp(a, b, op: op, count: count, dtype: dtype) }
    let db = try await device(b)
    let out = try output(count * dtype.byteSize)
    try check(
      hc_binary_op_scalar(
        ctx, hcOp(op), hcDType(dtype), db.pointer, a.toFloat(), dtype == .int64 ? a.toInt64() : 0, 1,
        out.pointer, count))
    return out
  }

  override open func elemwise(
    _ a: Tensor.Data, op: ElemwiseOp, scales: Tensor.Data?, count: Int, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype == .float16 || dtype == .float32 else {
      return try await super.elemwise(a, op: op, scales: scales, count: count, dtype: dtype)
    }
    let da = try await device(a)
    let ds = scales == nil ? nil : try await device(scales!)
    let out = try output(count * dtype.byteSize)
    try check(hc_elemwise(ctx, hcOp(op), hcDType(dtype), da.pointer, ds?.pointer, out.pointer, count))
    return out
  }

  override open func pow<T: NumericTensorElement>(
    _ a: Tensor.Data, _ b: T, scale: T, scales: Tensor.Data?, count: Int, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else {
      return try await super.pow(a, b, scale: scale, scales: scales, count: count, dtype: dtype)
    }
    let da = try await device(a)
    let ds = scales == nil ? nil : try await device(scales!)
    let out = try output(count * dtype.byteSize)
    let isInt = dtype == .int64
    try check(
      hc_pow(
        ctx, hcDType(dtype), da.pointer, b.toFloat(), scale.toFloat(), isInt ? b.toInt64() : 0,
        isInt ? scale.toInt64() : 0, ds?.pointer, out.pointer, count))
    return out
  }

  override open func reduce(
    _ a: Tensor.Data, op: ReduceOp, dims: ReduceDims, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    let da = try await device(a)  // (bool reduces as Float 0 / 1, like the CPU: Tensor.all / some)
    let outType: Tensor.DType = op.isIntOut ? .int64 : dtype
    let out = try output(dims.outCount * outType.byteSize)
    try check(
      hc_reduce(
        ctx, hcOp(op), hcDType(dtype), da.pointer, out.pointer, Int64(dims.outerCount),
        Int64(dims.reduceCount), Int64(dims.innerCount)))
    return out
  }

  override open func gather(
    _ a: Tensor.Data, _ s: ScatterGatherIndices, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    let (da, di) = (try await device(a), try await device(s.indices.data))
    var st = hcStrides(s.indices.strides)
    let out = try output(s.gatherOutCount * dtype.byteSize)
    let axis = s.axis
    // The gather of t / swap / move / PermuteAxes (Index.swift:238-266): indices from
    // axisPermutation that run along the gathered axis only. hc_permute moves the same bytes
    // without reading 8 bytes of index per element.
    if let meta = di.permutation, s.indices.strides.shape[axis] == meta.shape.product(),
      s.valueShape[axis] == meta.shape.product(),
      zip(s.indices.strides.shape, s.indices.strides.strides).enumerated().allSatisfy({ ax, e in
        e.0 == 1 || e.1 == (ax == axis ? 1 : 0)
      })
    {
      var perm = meta.permutation.map { Int64($0) }
      var shape = meta.shape.map { Int64($0) }
      let outer = s.valueShape[..<axis].product()
      if outer > 1 {
        perm = [0] + perm.map { $0 + 1 }
        shape = [Int64(outer)] + shape
      }
      if shape.count <= 8 {  // (more axes fall through to the index gather)
        try check(
          hc_permute(
            ctx, hcDType(dtype), da.pointer, perm, shape, Int32(shape.count),
            Int64(s.valueShape[(axis + 1)...].product()), out.pointer))
        return out
      }
    }
    try check(
      hc_gather(
        ctx, hcDType(dtype), da.pointer, di.pointer, &st, out.pointer,
        Int64(s.valueShape[..<axis].product()), Int64(s.valueShape[axis]),
        Int64(s.indices.strides.shape[axis]), Int64(s.valueShape[(axis + 1)...].product())))
    return out
  }

  /// The index vector depends on (permutation, shape) only and every permuted view rebuilds it
  /// (Index.swift:238-266): finished vectors are kept and shared (buffers are immutable), never
  /// evicted (a recorded graph may read them), and not added while recording.
  private struct PermutationKey: Hashable {
    let permutation: [Int]
    let shape: [Int]
  }
  private var permutationCache: [PermutationKey: HIPData] = [:]
  private var permutationCacheBytes = 0
  private let permutationCacheLock = NSLock()
  var isCapturing = false

  override open func axisPermutation(permutation: [Int], shape: [Int]) async throws -> Tensor.Data {
    let key = PermutationKey(permutation: permutation, shape: shape)
    if let hit = permutationCacheLock.withLock({ permutationCache[key] }) { return hit }
    let out = try output(shape.product() * Tensor.DType.int64.byteSize)
    let (perm, shp) = (permutation.map { Int64($0) }, shape.map { Int64($0) })
    try check(hc_axis_permutation(ctx, perm, shp, Int32(shape.count), out.pointer))
    out.permutation = (permutation, shape)
    permutationCacheLock.withLock {
      if !isCapturing && permutationCacheBytes + out.byteCount <= 256 << 20 {
        permutationCache[key] = out
        permutationCacheBytes += out.byteCount
      }
    }
    return out
  }

  // MARK: - the rest of a transformer forward pass

  override open func logSoftmax(_ a: Tensor.Data, dims: ReduceDims, dtype: Tensor.DType) async throws
    -> Tensor.Data
  {
    guard dtype == .float16 || dtype == .float32 else {
      return try await super.logSoftmax(a, dims: dims, dtype: dtype)
    }
    let da = try await device(a)
    let out = try output(dims.inCount * dtype.byteSize)
    try check(
      hc_log_softmax(
        ctx, hcDType(dtype), da.pointer, out.pointer, Int64(dims.outerCount), Int64(dims.reduceCount),
        Int64(dims.innerCount)))
    return out
  }

  /// Fused override of the base-class composition (Backend.swift:265-327), same arithmetic.
  override open func normalize<T: NumericTensorElement>(
    input: Tensor.Data, dims: ReduceDims, eps: T, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype == .float16 || dtype == .float32 else {
      return try await super.normalize(input: input, dims: dims, eps: eps, dtype: dtype)
    }
    let da = try await device(input)
    let out = try output(dims.inCount * dtype.byteSize)
    try check(
      hc_normalize(
        ctx, hcDType(dtype), da.pointer, out.pointer, Int64(dims.outerCount), Int64(dims.reduceCount),
        Int64(dims.innerCount), eps.toFloat()))
    return out
  }

  override open func cast(_ a: Tensor.Data, count: Int, inType: Tensor.DType, outType: Tensor.DType)
    async throws -> Tensor.Data
  {
    let da = try await device(a)
    let out = try output(count * outType.byteSize)
    try check(hc_cast(ctx, da.pointer, hcDType(inType), out.pointer, hcDType(outType), count))
    return out
  }

  override open func mulAdd(
    input: BroadcastData, coeff: BroadcastData, bias: BroadcastData, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else {
      return try await super.mulAdd(input: input, coeff: coeff, bias: bias, dtype: dtype)
    }
    let (di, dc, db) = (try await device(input.data), try await device(coeff.data), try await device(bias.data))
    var (si, sc, sb) = (hcStrides(input.strides), hcStrides(coeff.strides), hcStrides(bias.strides))
    let out = try output(input.strides.shape.product() * dtype.byteSize)
    try check(hc_mul_add(ctx, hcDType(dtype), di.pointer, &si, dc.pointer, &sc, db.pointer, &sb, out.pointer))
    return out
  }

  override open func addMul(
    input: BroadcastData, bias: BroadcastData, coeff: BroadcastData, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else {
      return try await super.addMul(input: input, bias: bias, coeff: coeff, dtype: dtype)
    }
    let (di, dc, db) = (try await device(input.data), try await device(coeff.data), try await device(bias.data))
    var (si, sc, sb) = (hcStrides(input.strides), hcStrides(coeff.strides), hcStrides(bias.strides))
    let out = try output(input.strides.shape.product() * dtype.byteSize)
    try check(hc_add_mul(ctx, hcDType(dtype), di.pointer, &si, db.pointer, &sb, dc.pointer, &sc, out.pointer))
    return out
  }

  override open func broadcast(_ a: BroadcastData, dtype: Tensor.DType) async throws -> Tensor.Data {
    let da = try await device(a.data)
    var sa = hcStrides(a.strides)
    let out = try output(a.strides.shape.product() * dtype.byteSize)
    try check(hc_broadcast(ctx, hcDType(dtype), da.pointer, &sa, out.pointer))
    return out
  }

  override open func compare(
    _ a: BroadcastData, _ b: BroadcastData, op: ComparisonOp, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    let (da, db) = (try await device(a.data), try await device(b.data))
    var (sa, sb) = (hcStrides(a.strides), hcStrides(b.strides))
    let out = try output(a.strides.shape.product())
    try check(hc_compare(ctx, hcOp(op), hcDType(dtype), da.pointer, &sa, db.pointer, &sb, out.pointer))
    return out
  }

  /// compare(Tensor.Data, T) / compare(T, Tensor.Data) (Backend.swift:468-486): the scalar is
  /// compared as Float, or as Int64 for int64 tensors (BackendCPU.swift:574-624).
  private func compareScalar<T: TensorElement>(
    _ a: Tensor.Data, _ b: T, scalarFirst: Bool, op: ComparisonOp, count: Int, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    let da = try await device(a)
    let out = try output(count)
    try check(
      hc_compare_scalar(
        ctx, hcOp(op), hcDType(dtype), da.pointer, b.toFloat(), dtype == .int64 ? b.toInt64() : 0,
        scalarFirst ? 1 : 0, out.pointer, count))
    return out
  }

  override open func compare<T: TensorElement>(
    _ a: Tensor.Data, _ b: T, op: ComparisonOp, count: Int, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    try await compareScalar(a, b, scalarFirst: false, op: op, count: count, dtype: dtype)
  }

  override open func compare<T: TensorElement>(
    _ a: T, _ b: Tensor.Data, op: ComparisonOp, count: Int, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    try await compareScalar(b, a, scalarFirst: true, op: op, count: count, dtype: dtype)
  }

  /// A TensorOrScalar operand as (device buffer, strides): a scalar becomes a 1-element constant
  /// with all-zero strides, which is what CPUBackend.tensorOrScalarData makes of it too.
  private func operand<T: TensorElement>(_ x: TensorOrScalar<T>, dtype: Tensor.DType) async throws
    -> (HIPData, hc_strides)
  {
    switch x {
    case .tensor(let t): return (try await device(t.data), hcStrides(t.strides))
    case .scalar(let v, let shape):
      let c = try await constant(v, count: 1, dtype: dtype)
      return (
        try await device(c),
        hcStrides(BroadcastStrides(shape: shape, strides: [Int](repeating: 0, count: shape.count)))
      )
    }
  }

  /// Backend.when (Backend.swift:633-641): mask ? a : b over the mask's broadcast shape.
  override open func when<T>(
    _ mask: BroadcastData, _ a: TensorOrScalar<T>, _ b: TensorOrScalar<T>, _: T.Type,
    dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    let dm = try await device(mask.data)
    var sm = hcStrides(mask.strides)
    var (da, sa) = try await operand(a, dtype: dtype)
    var (db, sb) = try await operand(b, dtype: dtype)
    let out = try output(mask.strides.shape.product() * dtype.byteSize)
    try check(hc_when(ctx, hcDType(dtype), dm.pointer, &sm, da.pointer, &sa, db.pointer, &sb, out.pointer))
    _ = (da, db)  // (the operands stay alive until the call has been enqueued)
    return out
  }

  /// Backend.concat (Backend.swift:777-784): input t contributes innerCounts[t] elements to each
  /// of the outerCount output rows.
  override open func concat(
    _ inputs: [Tensor.Data], outerCount: Int, innerCounts: [Int], dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    var buffers: [HIPData] = []
    for x in inputs { buffers.append(try await device(x)) }
    let pointers: [UnsafeRawPointer?] = buffers.map { UnsafeRawPointer($0.pointer) }
    let counts = innerCounts.map { Int64($0) }
    let out = try output(outerCount * innerCounts.reduce(0, +) * dtype.byteSize)
    try check(
      hc_concat(ctx, hcDType(dtype), pointers, counts, Int32(inputs.count), Int64(outerCount), out.pointer))
    return out
  }

  /// Backend.collection (Backend.swift:794-800): the element conversion stays the host's
  /// (CPUBackend.collection, BackendCPU.swift:1817-1829); the result is uploaded once, here,
  /// instead of at every op that reads it.
  override open func collection<T: TensorElement>(
    _ collection: some Collection<T>, reverse: Bool, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    try await device(try await super.collection(collection, reverse: reverse, dtype: dtype))
  }

  /// Backend.repeated (Backend.swift:590-606) as the broadcast it is defined as; CPUBackend
  /// overrides it with a host loop (BackendCPU.swift:1087-1106).
  override open func repeated(_ a: Tensor.Data, dims: RepeatDims, dtype: Tensor.DType) async throws
    -> Tensor.Data
  {
    try await broadcast(
      BroadcastData(
        strides: BroadcastStrides(
          shape: [dims.outerCount, dims.repeatCount, dims.innerCount],
          strides: [dims.innerCount, 0, 1]),
        data: a),
      dtype: dtype)
  }

  /// bitwiseOp(Tensor.Data, T) (Backend.swift:227-235): the scalar's bit pattern as a 1-element
  /// buffer with a zero stride.
  override open func bitwiseOp<T: TensorElementBitPattern>(
    _ a: Tensor.Data, _ b: T, op: BitwiseOp, count: Int, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    let bits = b.bitsForBitwiseOp
    guard bits.count == dtype.byteSize else {
      return try await super.bitwiseOp(a, b, op: op, count: count, dtype: dtype)
    }
    let da = try await device(a)
    let db = try output(bits.count)
    try bits.withUnsafeBytes { try check(hc_memcpy_h2d(ctx, db.pointer, $0.baseAddress, bits.count)) }
    var sa = hcStrides(BroadcastStrides(shape: [count], strides: [1]))
    var sb = hcStrides(BroadcastStrides(shape: [count], strides: [0]))
    let out = try output(count * dtype.byteSize)
    let kind: Int32 = op == .or ? 0 : op == .and ? 1 : 2
    try check(hc_bitwise_op(ctx, kind, hcDType(dtype), da.pointer, &sa, db.pointer, &sb, out.pointer))
    return out
  }

  override open func constant<T: TensorElement>(_ value: T, count: Int, dtype: Tensor.DType) async throws
    -> Tensor.Data
  {
    let out = try output(count * dtype.byteSize)
    try check(
      hc_fill(ctx, hcDType(dtype), value.toFloat(), dtype == .int64 ? value.toInt64() : 0, out.pointer, count))
    return out
  }

  override open func triangular(
    _ a: Tensor.Data, batch: Int, rows: Int, cols: Int, upper: Bool, offset: Int, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    let da = try await device(a)
    let out = try output(batch * rows * cols * dtype.byteSize)
    try check(
      hc_triangular(
        ctx, hcDType(dtype), da.pointer, out.pointer, Int64(batch), Int64(rows), Int64(cols),
        upper ? 1 : 0, Int64(offset)))
    return out
  }

  override open func bitwiseOp(
    _ a: BroadcastData, _ b: BroadcastData, op: BitwiseOp, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    let (da, db) = (try await device(a.data), try await device(b.data))
    var (sa, sb) = (hcStrides(a.strides), hcStrides(b.strides))
    let out = try output(a.strides.shape.product() * dtype.byteSize)
    let kind: Int32 = op == .or ? 0 : op == .and ? 1 : 2
    try check(hc_bitwise_op(ctx, kind, hcDType(dtype), da.pointer, &sa, db.pointer, &sb, out.pointer))
    return out
  }

  // MARK: - backward pass and optimizer

  override open func scatter(
    _ a: Tensor.Data, _ s: ScatterGatherIndices, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else { return try await super.scatter(a, s, dtype: dtype) }
    let (da, di) = (try await device(a), try await device(s.indices.data))
    var st = hcStrides(s.indices.strides)
    let out = try output(s.gatherInCount * dtype.byteSize)
    let axis = s.axis
    try check(
      hc_scatter(
        ctx, hcDType(dtype), da.pointer, di.pointer, &st, out.pointer,
        Int64(s.valueShape[..<axis].product()), Int64(s.valueShape[axis]),
        Int64(s.indices.strides.shape[axis]), Int64(s.valueShape[(axis + 1)...].product()),
        s.indicesAreUnique ? 1 : 0))
    return out
  }

  override open func logSoftmaxGrad(
    _ a: Tensor.Data, _ outGrad: Tensor.Data, dims: ReduceDims, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype == .float16 || dtype == .float32 else {
      return try await super.logSoftmaxGrad(a, outGrad, dims: dims, dtype: dtype)
    }
    let (da, dg) = (try await device(a), try await device(outGrad))
    let out = try output(dims.inCount * dtype.byteSize)
    try check(
      hc_log_softmax_grad(
        ctx, hcDType(dtype), da.pointer, dg.pointer, out.pointer, Int64(dims.outerCount),
        Int64(dims.reduceCount), Int64(dims.innerCount)))
    return out
  }

  private func cumulative(
    _ op: Int32, _ a: Tensor.Data, _ dims: ReduceDims, _ exclusive: Bool, _ reverse: Bool,
    _ dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    let da = try await device(a)
    let out = try output(dims.inCount * dtype.byteSize)
    try check(
      hc_cumulative(
        ctx, op, hcDType(dtype), da.pointer, out.pointer, Int64(dims.outerCount),
        Int64(dims.reduceCount), Int64(dims.innerCount), exclusive ? 1 : 0, reverse ? 1 : 0))
    return out
  }

  override open func cumulativeSum(
    _ a: Tensor.Data, dims: ReduceDims, exclusive: Bool, reverse: Bool, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else {
      return try await super.cumulativeSum(
        a, dims: dims, exclusive: exclusive, reverse: reverse, dtype: dtype)
    }
    return try await cumulative(0, a, dims, exclusive, reverse, dtype)
  }

  override open func cumulativeProd(
    _ a: Tensor.Data, dims: ReduceDims, exclusive: Bool, reverse: Bool, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else {
      return try await super.cumulativeProd(
        a, dims: dims, exclusive: exclusive, reverse: reverse, dtype: dtype)
    }
    return try await cumulative(1, a, dims, exclusive, reverse, dtype)
  }

  /// The device sort is stable whatever `stable` says.
  override open func argsort(
    _ a: Tensor.Data, dims: ReduceDims, descending: Bool, stable: Bool, dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else {
      return try await super.argsort(
        a, dims: dims, descending: descending, stable: stable, dtype: dtype)
    }
    let da = try await device(a)
    let out = try output(dims.inCount * 8)
    try check(
      hc_argsort(
        ctx, hcDType(dtype), da.pointer, out.pointer, Int64(dims.outerCount),
        Int64(dims.reduceCount), Int64(dims.innerCount), descending ? 1 : 0))
    return out
  }

  override open func clamp<T: NumericTensorElement>(
    _ a: BroadcastData, _: T.Type, min: TensorOrScalar<T>?, max: TensorOrScalar<T>?,
    dtype: Tensor.DType
  ) async throws -> Tensor.Data {
    guard dtype != .bool else { return try await super.clamp(a, T.self, min: min, max: max, dtype: dtype) }
    let da = try await device(a.data)
    var sa = hcStrides(a.strides)
    let lo = min == nil ? nil : try await operand(min!, dtype: dtype)
    let hi = max == nil ? nil : try await operand(max!, dtype: dtype)
    var (sl, sh) = (lo?.1 ?? sa, hi?.1 ?? sa)
    let out = try output(a.strides.shape.product() * dtype.byteSize)
    try withUnsafePointer(to: &sl) { pl in
      try withUnsafePointer(to: &sh) { ph in
        try check(
          hc_clamp(
            ctx, hcDType(dtype), da.pointer, &sa, lo?.0.pointer, lo == nil ? nil : pl, hi?.0.pointer,
            hi == nil ? nil : ph, out.pointer))
      }
    }
    return out
  }

  /// One fused kernel with the arithmetic of the base-class composition (Backend.swift:818-892).
  override open func adamW(
    param: Tensor.Data, grad: Tensor.Data, moment1: Tensor.Data, moment2: Tensor.Data,
    beta1: Float, beta2: Float, eps: Float, weightDecay: Float, lr: Float, step: Float, count: Int,
    dtype: Tensor.DType
  ) async throws -> (param: Tensor.Data, moment1: Tensor.Data, moment2: Tensor.Data) {
    guard dtype == .float16 || dtype == .float32 else {
      return try await super.adamW(
        param: param, grad: grad, moment1: moment1, moment2: moment2, beta1: beta1, beta2: beta2,
        eps: eps, weightDecay: weightDecay, lr: lr, step: step, count: count, dtype: dtype)
    }
    let (dp, dg) = (try await device(param), try await device(grad))
    let (d1, d2) = (try await device(moment1), try await device(moment2))
    let bytes = count * dtype.byteSize
    let (op, o1, o2) = (try output(bytes), try output(bytes), try output(bytes))
    try check(
      hc_adamw(
        ctx, hcDType(dtype), dp.pointer, dg.pointer, d1.pointer, d2.pointer, beta1, beta2, eps,
        weightDecay, lr, step, count, op.pointer, o1.pointer, o2.pointer))
    return (param: op, moment1: o1, moment2: o2)
  }

  // MARK: - recording and replay (no counterpart in Honeycrisp)

  /// A recorded sequence of backend calls; `launch()` replays all of them with one call.
  public final class Graph {
    let backend: HIPBackend
    let handle: OpaquePointer
    init(backend: HIPBackend, handle: OpaquePointer) { (self.backend, self.handle) = (backend, handle) }
    public func launch() throws { try backend.check(hc_graph_launch(backend.ctx, handle)) }
    /// Kernel launches and copies one replay issues (after the library's rewrite of the recording).
    public func nodeCount() throws -> Int {
      var n: Int = 0
      try backend.check(hc_graph_node_count(handle, &n))
      return n
    }
    deinit { _ = hc_graph_destroy(backend.ctx, handle) }
  }

  /// Runs `body` with every backend call recorded instead of executed. Inputs must already be
  /// on the device; tensors created inside keep their buffers reserved for the graph.
  public func capture(_ body: () async throws -> Void) async throws -> Graph {
    try check(hc_capture_begin(ctx))
    isCapturing = true
    defer { isCapturing = false }
    do { try await body() } catch {
      _ = hc_capture_abort(ctx)
      throw error
    }
    var handle: OpaquePointer?
    try check(hc_capture_end(ctx, &handle))
    return Graph(backend: self, handle: handle!)
  }
}

// Enum orders match include/hchip.h by construction of that header.
private func hcOp(_ op: NumericBinaryOp) -> Int32 {
  switch op { case .add: 0; case .mul: 1; case .sub: 2; case .div: 3; case .mod: 4 }
}
private func hcOp(_ op: ReduceOp) -> Int32 {
  switch op { case .sum: 0; case .prod: 1; case .argmax: 2; case .argmin: 3 }
}
private func hcOp(_ op: ComparisonOp) -> Int32 {
  switch op {
  case .equal: 0; case .notEqual: 1; case .less: 2; case .lessEqual: 3; case .greater: 4; case .greaterEqual: 5
  }
}
private func hcOp(_ op: ElemwiseOp) -> Int32 {
  switch op {
  case .sin: 0; case .cos: 1; case .minusSin: 2; case .tan: 3; case .tanGrad: 4; case .atan: 5
  case .atanGrad: 6; case .acos: 7; case .acosGrad: 8; case .asin: 9; case .asinGrad: 10; case .exp: 11
  case .log: 12; case .recip: 13; case .sigmoid: 14; case .sigmoidGrad: 15; case .relu: 16
  case .reluGrad: 17; case .abs: 18; case .absGrad: 19; case .geluApprox: 20; case .geluApproxGrad: 21
  case .geluExact: 22; case .geluExactGrad: 23; case .erf: 24; case .erfGrad: 25; case .floor: 26
  case .ceil: 27; case .round: 28
  }
}
