//
//  HIP.swift
//  DL4S
//
//  An MI355X (gfx950) device for DL4S: `Tensor<Float, HIP>`.
//
//  This file belongs inside the DL4S module, next to Engine/GPU/GPU.swift: `Buffer.memory`, `Buffer.init(memory:)`,
//  `ShapedBuffer.init(values:shape:)` and `Tensor.init(using:context:)` are internal (Engine/Buffer.swift:31,97,
//  Tensor/Tensor.swift:164).  It binds the C ABI of libdl4s_hip.so through the system-library target CDL4SHIP.
//
//  Every requirement of DeviceType / MemoryOperatorsType / EngineType (Engine/Engine.swift:30-581) is present.  The ones
//  the attention path and its callers use run HIP kernels; the rest trap, like every method of the Metal stub does
//  (Engine/GPU/GPU.swift:135-381) - they are marked unavailable, never faked.  The engine implements Float only; every
//  entry point traps for another element type.
//

import Foundation
import CDL4SHIP

// MARK: Device

/// Device memory handle: a raw device address.  An offset view is plain pointer arithmetic and is never freed.
public struct HIPBuffer: Hashable {
    var ptr: UnsafeMutableRawPointer
}

public struct HIP: DeviceType {
    public typealias Memory = HIPMemory
    public typealias Engine = HIPEngine

    /// One context (GPU, stream, pooled allocator) per process.  The environment variable DL4S_HIP_DEVICE selects the GPU.
    static let context: OpaquePointer = {
        let ordinal = ProcessInfo.processInfo.environment["DL4S_HIP_DEVICE"].flatMap { Int32($0) } ?? 0
        var created: OpaquePointer? = nil
        let status = dl4s_hip_create(ordinal, &created)
        guard status == 0, let context = created else {
            fatalError("dl4s_hip_create: \(String(cString: dl4s_hip_last_error()))")
        }
        return context
    }()

    /// The fused attention hook skips key tiles that its mask blocks entirely.  That is exact while keys and values are
    /// finite at blocked positions; the reference multiplies them by a weight of exactly zero, so a NaN or Inf there reaches
    /// its output and not this one's.  Set to true to visit every tile (DL4S_SDPA_STRICT): the reference's results down to
    /// `0 * NaN`, at about twice the time under a causal mask.
    public static var strictMasks = false

    /// Waits for everything enqueued so far (benchmarks; `elements`, `item` and every device-to-host copy wait by themselves).
    public static func synchronize() {
        hipCheck(dl4s_hip_sync(context))
    }
}

/// The reference traps on contract violations (precondition / fatalError); the C ABI returns a status and a message.
@inline(__always)
func hipCheck(_ status: Int32, _ function: StaticString = #function) {
    if status != 0 {
        fatalError("\(function): \(String(cString: dl4s_hip_last_error()))")
    }
}

// MARK: Memory

public struct HIPMemory: MemoryOperatorsType {
    public typealias Device = HIP
    public typealias RawBuffer = HIPBuffer

    @inline(__always)
    static func strides(from shape: [Int]) -> [Int] {
        var strides = [Int](repeating: 1, count: shape.count)
        for i in stride(from: shape.count - 2, through: 0, by: -1) {
            strides[i] = strides[i + 1] * shape[i + 1]
        }
        return strides
    }

    /// Device address of a buffer of 4-byte elements (the copy kernels do not look at the values).
    @inline(__always)
    static func words<Element>(_ buffer: Buffer<Element, HIP>) -> UnsafeMutablePointer<Float> {
        precondition(MemoryLayout<Element>.stride == 4, "HIP slices are implemented for 4-byte elements")
        return buffer.memory.ptr.assumingMemoryBound(to: Float.self)
    }

    public static func allocateBuffer<Element>(withCapacity capacity: Int, type: Element.Type) -> Buffer<Element, HIP> {
        var raw: UnsafeMutableRawPointer? = nil
        hipCheck(dl4s_hip_alloc(HIP.context, capacity * MemoryLayout<Element>.stride, &raw))
        return Buffer<Element, HIP>(memory: HIPBuffer(ptr: raw!))
    }

    public static func allocateBuffer<Element>(withShape shape: [Int], type: Element.Type) -> ShapedBuffer<Element, HIP> {
        return ShapedBuffer(values: allocateBuffer(withCapacity: shape.reduce(1, *), type: Element.self), shape: shape)
    }

    /// Stream-ordered: the block returns to the library's pool at once, later work on the stream may reuse it
    /// (TensorHandle.deinit frees right after the last use was enqueued, Tensor/Tensor.swift:38-42).
    public static func free<Element>(_ buffer: Buffer<Element, HIP>) {
        forgetPreparedMasks(in: buffer)
        hipCheck(dl4s_hip_free(HIP.context, buffer.memory.ptr))
    }

    /// What the fused attention calls remember about mask buffers (HIPPreparedMasks) describes the buffers' values: it goes
    /// when the allocation is freed or written through this type.
    @inline(__always)
    static func forgetPreparedMasks<Element>(in buffer: Buffer<Element, HIP>) {
        if HIPPreparedMasks.entries.isEmpty { return }
        var bytes = 0
        if dl4s_hip_get_size(HIP.context, buffer.memory.ptr, &bytes) == 0 {
            HIPPreparedMasks.forget(from: buffer.memory.ptr, bytes: bytes)
        }
    }

    public static func free<Element>(_ buffer: ShapedBuffer<Element, HIP>) {
        free(buffer.values)
    }

    public static func assign<Element>(from source: UnsafeBufferPointer<Element>, to destination: Buffer<Element, HIP>, count: Int) {
        forgetPreparedMasks(in: destination)
        hipCheck(dl4s_hip_assign_h2d(HIP.context, destination.memory.ptr, source.baseAddress, count * MemoryLayout<Element>.stride))
    }

    public static func assign<Element>(from source: Buffer<Element, HIP>, to destination: Buffer<Element, HIP>, count: Int) {
        forgetPreparedMasks(in: destination)
        hipCheck(dl4s_hip_assign_d2d(HIP.context, destination.memory.ptr, source.memory.ptr, count * MemoryLayout<Element>.stride))
    }

    public static func assign<Element>(from source: Buffer<Element, HIP>, to destination: UnsafeMutableBufferPointer<Element>, count: Int) {
        hipCheck(dl4s_hip_assign_d2h(HIP.context, destination.baseAddress, source.memory.ptr, count * MemoryLayout<Element>.stride))
    }

    public static func getValue<Element>(from source: Buffer<Element, HIP>) -> Element {
        let host = UnsafeMutableBufferPointer<Element>.allocate(capacity: 1)
        defer { host.deallocate() }
        assign(from: source, to: host, count: 1)
        return host[0]
    }

    /// Elements from the buffer's address to the end of its allocation (also for offset views, Engine/CPU/CPU.swift:219-221).
    public static func getSize<Element>(of buffer: Buffer<Element, HIP>) -> Int {
        var bytes = 0
        hipCheck(dl4s_hip_get_size(HIP.context, buffer.memory.ptr, &bytes))
        return bytes / MemoryLayout<Element>.stride
    }

    public static func get<Element>(slice: [Int?], of buffer: Buffer<Element, HIP>, with shape: [Int]) -> (Buffer<Element, HIP>, Bool, [Int]) {
        precondition(slice.count <= shape.count, "Index must be smaller than or equal to vector size")
        // an index that ends in nil entries reads whole trailing axes (Engine/CPU/CPU.swift:140-141)
        let trimmed = Array(slice.reversed().drop(while: { $0 == nil }).reversed())
        let strides = HIPMemory.strides(from: shape)
        if !trimmed.contains(where: { $0 == nil }) {
            // a pure prefix index: an offset into the same storage, no copy (Engine/CPU/CPU.swift:146-157)
            let offset = zip(trimmed, strides).map { $0.0! * $0.1 }.reduce(0, +)
            return (advance(buffer: buffer, by: offset), false, Array(shape.dropFirst(trimmed.count)))
        }
        let padded = trimmed + [Int?](repeating: nil, count: shape.count - trimmed.count)
        let start = padded.map { Int64($0 ?? 0) }
        let extent = zip(padded, shape).map { $0.0 == nil ? Int64($0.1) : Int64(1) }
        let resultShape = zip(padded, shape).compactMap { $0.0 == nil ? $0.1 : nil }
        let result = allocateBuffer(withCapacity: resultShape.reduce(1, *), type: Element.self)
        hipCheck(dl4s_hip_subscript_read_f32(HIP.context, words(buffer), shape.map { Int64($0) }, Int32(shape.count), start, extent, words(result)))
        return (result, true, resultShape)
    }

    public static func get<Element>(slice: [(CountableRange<Int>)?], of buffer: Buffer<Element, HIP>, with shape: [Int]) -> (Buffer<Element, HIP>, Bool, [Int]) {
        precondition(slice.count <= shape.count, "Index must be smaller than or equal to vector size")
        let padded = slice + [CountableRange<Int>?](repeating: nil, count: shape.count - slice.count)
        let start = padded.map { Int64($0?.lowerBound ?? 0) }
        let resultShape = zip(padded, shape).map { $0.0?.count ?? $0.1 }
        let result = allocateBuffer(withCapacity: resultShape.reduce(1, *), type: Element.self)
        hipCheck(dl4s_hip_subscript_read_f32(HIP.context, words(buffer), shape.map { Int64($0) }, Int32(shape.count), start,
                                             resultShape.map { Int64($0) }, words(result)))
        return (result, true, resultShape)
    }

    public static func set<Element>(slice: [Int?], of buffer: Buffer<Element, HIP>, with dstShape: [Int], from source: Buffer<Element, HIP>, with sourceShape: [Int]) {
        forgetPreparedMasks(in: buffer)
        let countDelta = dstShape.count - slice.filter { $0 != nil }.count
        precondition(sourceShape.count == countDelta, "Dimensionality of source must be equal to dimensionality of destination minus number of knowns in slice")
        let padded = slice + [Int?](repeating: nil, count: dstShape.count - slice.count)
        let start = padded.map { Int64($0 ?? 0) }
        let extent = zip(padded, dstShape).map { $0.0 == nil ? Int64($0.1) : Int64(1) }
        hipCheck(dl4s_hip_subscript_write_f32(HIP.context, words(source), words(buffer), dstShape.map { Int64($0) }, Int32(dstShape.count), start, extent))
    }

    public static func set<Element>(slice: [Range<Int>?], of buffer: Buffer<Element, HIP>, with dstShape: [Int], from source: Buffer<Element, HIP>, with sourceShape: [Int]) {
        forgetPreparedMasks(in: buffer)
        precondition(sourceShape.count == dstShape.count, "Dimensionality of source must be equal to dimensionality of destination")
        let padded = slice + [Range<Int>?](repeating: nil, count: dstShape.count - slice.count)
        let start = padded.map { Int64($0?.lowerBound ?? 0) }
        let extent = zip(padded, dstShape).map { Int64($0.0?.count ?? $0.1) }
        hipCheck(dl4s_hip_subscript_write_f32(HIP.context, words(source), words(buffer), dstShape.map { Int64($0) }, Int32(dstShape.count), start, extent))
    }

    public static func setPointee<Element>(of buffer: Buffer<Element, HIP>, to newValue: Element) {
        forgetPreparedMasks(in: buffer)
        var value = newValue
        withUnsafePointer(to: &value) { pointer in
            hipCheck(dl4s_hip_assign_h2d(HIP.context, buffer.memory.ptr, pointer, MemoryLayout<Element>.stride))
        }
    }

    public static func advance<Element>(buffer: Buffer<Element, HIP>, by advancement: Int) -> Buffer<Element, HIP> {
        return Buffer<Element, HIP>(memory: HIPBuffer(ptr: buffer.memory.ptr + advancement * MemoryLayout<Element>.stride))
    }
}

// MARK: Engine

public struct HIPEngine: EngineType {
    public typealias Device = HIP

    @inline(__always)
    static func f<N>(_ buffer: Buffer<N, HIP>, _ function: StaticString = #function) -> UnsafeMutablePointer<Float> {
        precondition(N.self == Float.self, "\(function): the HIP engine implements Float only")
        return buffer.memory.ptr.assumingMemoryBound(to: Float.self)
    }

    @inline(__always)
    static func f<N>(_ buffer: ShapedBuffer<N, HIP>, _ function: StaticString = #function) -> UnsafeMutablePointer<Float> {
        return f(buffer.values, function)
    }

    @inline(__always)
    static func dims(_ shape: [Int]) -> [Int64] {
        return shape.map { Int64($0) }
    }

    static func unavailable(_ function: StaticString = #function) -> Never {
        fatalError("\(function) is not available for HIP")
    }

    // MARK: same-shape element-wise operations

    public static func fill<N: NumericType>(value: N, result: Buffer<N, HIP>, count: Int) {
        hipCheck(dl4s_hip_fill_f32(HIP.context, value as! Float, f(result), Int64(count)))
    }

    public static func vAdd<N: NumericType>(lhs: Buffer<N, HIP>, rhs: Buffer<N, HIP>, result: Buffer<N, HIP>, count: Int) {
        hipCheck(dl4s_hip_vadd_f32(HIP.context, f(lhs), f(rhs), f(result), Int64(count)))
    }

    public static func vNeg<N: NumericType>(val: Buffer<N, HIP>, result: Buffer<N, HIP>, count: Int) {
        hipCheck(dl4s_hip_vneg_f32(HIP.context, f(val), f(result), Int64(count)))
    }

    public static func vSub<N: NumericType>(lhs: Buffer<N, HIP>, rhs: Buffer<N, HIP>, result: Buffer<N, HIP>, count: Int) {
        hipCheck(dl4s_hip_vsub_f32(HIP.context, f(lhs), f(rhs), f(result), Int64(count)))
    }

    public static func vMul<N: NumericType>(lhs: Buffer<N, HIP>, rhs: Buffer<N, HIP>, result: Buffer<N, HIP>, count: Int) {
        hipCheck(dl4s_hip_vmul_f32(HIP.context, f(lhs), f(rhs), f(result), Int64(count)))
    }

    public static func vDiv<N: NumericType>(lhs: Buffer<N, HIP>, rhs: Buffer<N, HIP>, result: Buffer<N, HIP>, count: Int) {
        hipCheck(dl4s_hip_vdiv_f32(HIP.context, f(lhs), f(rhs), f(result), Int64(count)))
    }

    // MARK: matrix operations

    public static func gemm<N: NumericType>(lhs: ShapedBuffer<N, HIP>, rhs: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, alpha: N, beta: N, transposeFirst: Bool, transposeSecond: Bool) {
        precondition(lhs.dim == 2 && rhs.dim == 2 && result.dim == 2, "gemm operands must be matrices")
        hipCheck(dl4s_hip_gemm_f32(HIP.context, f(lhs), Int64(lhs.shape[0]), Int64(lhs.shape[1]), f(rhs), Int64(rhs.shape[0]), Int64(rhs.shape[1]),
                                   f(result), alpha as! Float, beta as! Float, transposeFirst ? 1 : 0, transposeSecond ? 1 : 0))
    }

    public static func band<N: NumericType>(buffer: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, belowDiagonal: Int?, aboveDiagonal: Int?) {
        precondition(buffer.dim == 2 && buffer.shape == result.shape, "band operands must be matrices of one shape")
        hipCheck(dl4s_hip_band_f32(HIP.context, f(buffer), f(result), Int64(buffer.shape[0]), Int64(buffer.shape[1]),
                                   belowDiagonal == nil ? 0 : 1, Int64(belowDiagonal ?? 0), aboveDiagonal == nil ? 0 : 1, Int64(aboveDiagonal ?? 0)))
    }

    // MARK: broadcasting operations

    @inline(__always)
    static func broadcast<N: NumericType>(_ op: dl4s_binary_op, _ lhs: ShapedBuffer<N, HIP>, _ rhs: ShapedBuffer<N, HIP>, _ result: ShapedBuffer<N, HIP>, _ function: StaticString = #function) {
        hipCheck(dl4s_hip_broadcast_f32(HIP.context, Int32(op.rawValue), f(lhs, function), dims(lhs.shape), Int32(lhs.dim),
                                        f(rhs, function), dims(rhs.shape), Int32(rhs.dim), f(result, function)), function)
    }

    public static func broadcastAdd<N: NumericType>(lhs: ShapedBuffer<N, HIP>, rhs: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        broadcast(DL4S_OP_ADD, lhs, rhs, result)
    }

    public static func broadcastSub<N: NumericType>(lhs: ShapedBuffer<N, HIP>, rhs: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        broadcast(DL4S_OP_SUB, lhs, rhs, result)
    }

    public static func broadcastMul<N: NumericType>(lhs: ShapedBuffer<N, HIP>, rhs: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        broadcast(DL4S_OP_MUL, lhs, rhs, result)
    }

    public static func broadcastDiv<N: NumericType>(lhs: ShapedBuffer<N, HIP>, rhs: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        broadcast(DL4S_OP_DIV, lhs, rhs, result)
    }

    // MARK: reductions

    public static func reduceSum<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, axis: Int) {
        reduceSum(values: values, result: result, axes: [axis])
    }

    public static func reduceSum<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, axes: [Int]) {
        hipCheck(dl4s_hip_reduce_sum_f32(HIP.context, f(values), dims(values.shape), Int32(values.dim), axes.map { Int32($0) }, Int32(axes.count), f(result)))
    }

    public static func reduceMax<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, context: ShapedBuffer<Int32, HIP>?, axis: Int) {
        // the forward pass of softmax passes no context (Tensor/Operators/Reduce.swift:248-249); the argmax context is
        // what the backward pass of reduceMax scatters through
        precondition(context == nil, "reduceMax with an argmax context is not available for HIP")
        hipCheck(dl4s_hip_reduce_max_f32(HIP.context, f(values), dims(values.shape), Int32(values.dim), Int32(axis), f(result)))
    }

    public static func sum<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        if values.dim == 0 {
            HIPMemory.assign(from: values.values, to: result.values, count: 1)
        } else {
            reduceSum(values: values, result: result, axes: Array(0 ..< values.dim))
        }
    }

    @discardableResult
    public static func max<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) -> Int {
        let (index, value) = argmax(values: values.values, count: values.shape.reduce(1, *))
        HIPMemory.setPointee(of: result.values, to: value)
        return index
    }

    /// Index of the first maximum; NaN is never selected; (0, -infinity) for an empty buffer (Engine/CPU/Numeric/CPUFloat.swift:294-318).
    /// Waits for the stream: the result is a host value.
    public static func argmax<N: NumericType>(values: Buffer<N, HIP>, count: Int) -> (Int, N) {
        var index: Int64 = 0
        var value: Float = 0
        hipCheck(dl4s_hip_argmax_f32(HIP.context, f(values), Int64(count), &index, &value))
        return (Int(index), value as! N)
    }

    // MARK: element-wise functions

    public static func exp<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        hipCheck(dl4s_hip_exp_f32(HIP.context, f(values), f(result), Int64(values.shape.reduce(1, *))))
    }

    public static func log<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        hipCheck(dl4s_hip_log_f32(HIP.context, f(values), f(result), Int64(values.shape.reduce(1, *))))
    }

    public static func sqrt<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        hipCheck(dl4s_hip_sqrt_f32(HIP.context, f(values), f(result), Int64(values.shape.reduce(1, *))))
    }

    public static func relu<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        hipCheck(dl4s_hip_relu_f32(HIP.context, f(values), f(result), Int64(values.shape.reduce(1, *))))
    }

    public static func sin<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        hipCheck(dl4s_hip_sin_f32(HIP.context, f(values), f(result), Int64(values.shape.reduce(1, *))))
    }

    public static func cos<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        hipCheck(dl4s_hip_cos_f32(HIP.context, f(values), f(result), Int64(values.shape.reduce(1, *))))
    }

    public static func tanh<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        hipCheck(dl4s_hip_tanh_f32(HIP.context, f(values), f(result), Int64(values.shape.reduce(1, *))))
    }

    // MARK: layout operations

    /// Source axis i becomes destination axis arangement[i] (Engine/CPU/CPUEngine.swift:897-935).
    public static func permuteAxes<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, arangement: [Int]) {
        hipCheck(dl4s_hip_permute_axes_f32(HIP.context, f(values), dims(values.shape), Int32(values.dim), arangement.map { Int32($0) }, f(result)))
    }

    public static func subscriptRead<N>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, index: [Int?]) {
        // Engine/CPU/CPUEngine.swift:973-981: get(slice:) then a copy into result
        let (buffer, isCopy, shape) = HIPMemory.get(slice: index, of: values.values, with: values.shape)
        HIPMemory.assign(from: buffer, to: result.values, count: shape.reduce(1, *))
        if isCopy {
            HIPMemory.free(buffer)
        }
    }

    /// The CPU engine leaves this one unimplemented (Engine/CPU/CPUEngine.swift:983-985); here it is set(slice:).
    public static func subscriptWrite<N>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, index: [Int?]) {
        HIPMemory.set(slice: index, of: result.values, with: result.shape, from: values.values, with: values.shape)
    }

    /// Tensor/Operators/Stack.swift:79-98; buffer i is [outer, its extent on the axis times the trailing extents].
    public static func stack<N>(buffers: [ShapedBuffer<N, HIP>], result: ShapedBuffer<N, HIP>, axis: Int) {
        precondition(N.self == Float.self, "the HIP engine implements Float only")
        let outer = result.shape.prefix(axis).reduce(1, *)
        let chunks = buffers.map { Int64($0.shape.suffix(from: axis).reduce(1, *)) }
        let sources: [UnsafePointer<Float>?] = buffers.map { UnsafePointer($0.values.memory.ptr.assumingMemoryBound(to: Float.self)) }
        hipCheck(dl4s_hip_stack_axis_f32(HIP.context, sources, chunks, Int64(buffers.count), Int64(outer),
                                         result.values.memory.ptr.assumingMemoryBound(to: Float.self)))
    }
}

// MARK: requirements that neither the attention path nor its callers use

extension HIPEngine {
    public static func fillDiagonal<N: NumericType>(values: ShapedBuffer<N, HIP>, target: ShapedBuffer<N, HIP>) { unavailable() }
    public static func fillDiagonal<N: NumericType>(value: N, target: ShapedBuffer<N, HIP>) { unavailable() }
    public static func extractDiagonal<N: NumericType>(values: ShapedBuffer<N, HIP>, target: ShapedBuffer<N, HIP>) { unavailable() }

    public static func reduceMin<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, context: ShapedBuffer<Int32, HIP>?, axis: Int) { unavailable() }
    public static func reduceMean<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, axis: Int) { unavailable() }
    public static func reduceMax<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, context: ShapedBuffer<Int32, HIP>?, axes: [Int]) { unavailable() }
    public static func reduceMin<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, context: ShapedBuffer<Int32, HIP>?, axes: [Int]) { unavailable() }
    public static func reduceMean<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, axes: [Int]) { unavailable() }
    public static func mean<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) { unavailable() }
    @discardableResult
    public static func min<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) -> Int { unavailable() }

    public static func heaviside<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) { unavailable() }
    public static func tan<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) { unavailable() }
    public static func sinh<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) { unavailable() }
    public static func cosh<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) { unavailable() }

    public static func max<N: NumericType>(_ lhs: ShapedBuffer<N, HIP>, _ rhs: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) { unavailable() }
    public static func max<N: NumericType>(_ lhs: ShapedBuffer<N, HIP>, _ rhs: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, context: ShapedBuffer<N, HIP>) { unavailable() }
    public static func min<N: NumericType>(_ lhs: ShapedBuffer<N, HIP>, _ rhs: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) { unavailable() }
    public static func min<N: NumericType>(_ lhs: ShapedBuffer<N, HIP>, _ rhs: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, context: ShapedBuffer<N, HIP>) { unavailable() }

    public static func scatter<N: NumericType>(reduced: ShapedBuffer<N, HIP>, context: ShapedBuffer<Int32, HIP>, result: ShapedBuffer<N, HIP>, axis: Int, ignoreIndex: Int32) { unavailable() }
    public static func gather<N: NumericType>(expanded: ShapedBuffer<N, HIP>, context: ShapedBuffer<Int32, HIP>, result: ShapedBuffer<N, HIP>, axis: Int, ignoreIndex: Int32) { unavailable() }

    public static func permuteAxesAdd<N: NumericType>(values: ShapedBuffer<N, HIP>, add: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, arangement: [Int]) { unavailable() }
    public static func subscriptReadAdd<N: NumericType>(values: ShapedBuffer<N, HIP>, add: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, index: [Int?]) { unavailable() }
    public static func subscriptWriteAdd<N: NumericType>(values: ShapedBuffer<N, HIP>, add: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, index: [Int?]) { unavailable() }
    public static func reverse<N>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) { unavailable() }
    public static func reverseAdd<N: NumericType>(values: ShapedBuffer<N, HIP>, add: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) { unavailable() }
    public static func unstackAdd<N: NumericType>(stacked: ShapedBuffer<N, HIP>, add: [ShapedBuffer<N, HIP>], result: [ShapedBuffer<N, HIP>], axis: Int) { unavailable() }
    public static func unstack<N: NumericType>(stacked: ShapedBuffer<N, HIP>, result: [ShapedBuffer<N, HIP>], axis: Int) { unavailable() }
    public static func arange<N: NumericType>(lowerBound: N, upperBound: N, result: ShapedBuffer<N, HIP>) { unavailable() }

    public static func img2col<N: NumericType>(values: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>, kernelWidth: Int, kernelHeight: Int, padding: Int, stride: Int) { unavailable() }
    public static func col2img<N: NumericType>(matrix: ShapedBuffer<N, HIP>, image: ShapedBuffer<N, HIP>, kernelWidth: Int, kernelHeight: Int, padding: Int, stride: Int) { unavailable() }
}
