//
//  HIPFusedAttention.swift
//  DL4S
//
//  EngineType has no attention operation and the layers are generic structs, so a backend cannot take over
//  ScaledDotProductAttention without a hook.  This file holds the hook's defaults for every engine, its implementation
//  for HIPEngine, and the fused path of the layer; patches/Engine.swift.patch declares the four requirements in
//  EngineType and patches/ScaledDotProductAttention.swift.patch adds the lines at the top of
//  ScaledDotProductAttention.callAsFunction (NN/Models/Transformer/ScaledDotProductAttention.swift:43-64) that use it.
//  Engines that keep the defaults (CPU) run the operator sequence as before, which on HIP stays available as the
//  cross-check of the fused kernels.
//

import Foundation
import CDL4SHIP

// The hook: four static requirements added to EngineType (patches/Engine.swift.patch) with the defaults below, so that
// `Device.Engine.hasFusedAttention` is an ordinary static dispatch and every existing engine keeps compiling unchanged.
//
//   fusedAttention             softmax((q / temperature) . k^T - mask * 1e9, axis: keys) . v in one call.
//                              q [batch, heads, queries, keyDim], k [batch, heads, keys, keyDim], v [batch, heads, keys, valueDim],
//                              mask broadcastable to [batch, heads, queries, keys] with 1 = blocked,
//                              result [batch, heads, queries, valueDim]
//   fusedAttentionForwardStats the same, also leaving two statistics per query row in stats [batch, heads, queries, 2]
//   fusedAttentionBackward     gradients of q, k and v for the upstream gradient of result (the mask takes none)
extension EngineType {
    public static var hasFusedAttention: Bool { return false }

    public static func fusedAttention<N: NumericType>(q: ShapedBuffer<N, Device>, k: ShapedBuffer<N, Device>, v: ShapedBuffer<N, Device>,
                                                      mask: ShapedBuffer<N, Device>?, result: ShapedBuffer<N, Device>, temperature: N) {
        fatalError("\(#function) is not available for \(self)")
    }

    public static func fusedAttentionForwardStats<N: NumericType>(q: ShapedBuffer<N, Device>, k: ShapedBuffer<N, Device>, v: ShapedBuffer<N, Device>,
                                                                  mask: ShapedBuffer<N, Device>?, result: ShapedBuffer<N, Device>,
                                                                  stats: ShapedBuffer<N, Device>, temperature: N) {
        fatalError("\(#function) is not available for \(self)")
    }

    public static func fusedAttentionBackward<N: NumericType>(q: ShapedBuffer<N, Device>, k: ShapedBuffer<N, Device>, v: ShapedBuffer<N, Device>,
                                                              mask: ShapedBuffer<N, Device>?, result: ShapedBuffer<N, Device>,
                                                              stats: ShapedBuffer<N, Device>, resultGradient: ShapedBuffer<N, Device>,
                                                              qGradient: ShapedBuffer<N, Device>, kGradient: ShapedBuffer<N, Device>,
                                                              vGradient: ShapedBuffer<N, Device>, temperature: N) {
        fatalError("\(#function) is not available for \(self)")
    }
}

extension HIPEngine {
    public static var hasFusedAttention: Bool { return true }

    /// The layer's dense float mask as the library's descriptor: right-aligned to [batch, heads, queries, keys], size-1 axes
    /// broadcast (Util.swift:40-45).
    static func denseDescriptor<N: NumericType>(for mask: ShapedBuffer<N, HIP>) -> dl4s_mask_desc {
        precondition(mask.dim <= 4, "attention masks have at most 4 axes")
        let padded = [Int](repeating: 1, count: 4 - mask.dim) + mask.shape
        var descriptor = dl4s_mask_desc()
        descriptor.kind = Int32(DL4S_MASK_DENSE_F32.rawValue)
        descriptor.dense = UnsafePointer(f(mask))
        descriptor.shape = (Int64(padded[0]), Int64(padded[1]), Int64(padded[2]), Int64(padded[3]))
        return descriptor
    }

    /// The descriptor an attention call passes for `mask`.  Every layer of a model receives the one mask tensor its model
    /// built (TransformerEncoder.swift:63, TransformerDecoder.swift:53-54), so a mask buffer is looked at once
    /// (`HIPPreparedMasks`): when its values are exactly a causal and / or key-length mask - what makeEncoderMasks and
    /// makeDecoderMasks build, TransformerUtil.swift:29-50 - the calls get the structured descriptor and read no mask
    /// values; any other mask keeps its dense descriptor together with its tile classes, so that later calls skip the
    /// classification.  The results are the bits of the dense descriptor either way.
    static func descriptor<N: NumericType>(for mask: ShapedBuffer<N, HIP>?, batchSize: Int, heads: Int, queryCount: Int, keyCount: Int) -> dl4s_mask_desc {
        guard let mask = mask else {
            var none = dl4s_mask_desc()
            none.kind = Int32(DL4S_MASK_NONE.rawValue)
            return none
        }
        return HIPPreparedMasks.descriptor(for: mask, batchSize: batchSize, heads: heads, queryCount: queryCount, keyCount: keyCount)
    }

    static var attentionFlags: UInt32 {
        return HIP.strictMasks ? DL4S_SDPA_STRICT : 0
    }

    public static func fusedAttention<N: NumericType>(q: ShapedBuffer<N, HIP>, k: ShapedBuffer<N, HIP>, v: ShapedBuffer<N, HIP>,
                                                      mask: ShapedBuffer<N, HIP>?, result: ShapedBuffer<N, HIP>, temperature: N) {
        precondition(q.dim == 4 && k.dim == 4 && v.dim == 4)
        var descriptor = self.descriptor(for: mask, batchSize: q.shape[0], heads: q.shape[1], queryCount: q.shape[2], keyCount: k.shape[2])
        // the reference forms the reciprocal once in Float and multiplies (Engine/CPU/CPUEngine.swift:635)
        let reciprocal = Float(1) / (temperature as! Float)
        hipCheck(dl4s_hip_sdpa_fwd_f32(HIP.context, f(q), f(k), f(v), f(result),
                                       Int64(q.shape[0]), Int64(q.shape[1]), Int64(q.shape[2]), Int64(k.shape[2]),
                                       Int64(q.shape[3]), Int64(v.shape[3]), reciprocal,
                                       descriptor.kind == Int32(DL4S_MASK_NONE.rawValue) ? nil : &descriptor, attentionFlags))
    }

    public static func fusedAttentionForwardStats<N: NumericType>(q: ShapedBuffer<N, HIP>, k: ShapedBuffer<N, HIP>, v: ShapedBuffer<N, HIP>,
                                                                  mask: ShapedBuffer<N, HIP>?, result: ShapedBuffer<N, HIP>,
                                                                  stats: ShapedBuffer<N, HIP>, temperature: N) {
        precondition(q.dim == 4 && k.dim == 4 && v.dim == 4 && q.shape[3] == v.shape[3], "the training form needs keyDim == valueDim")
        var descriptor = self.descriptor(for: mask, batchSize: q.shape[0], heads: q.shape[1], queryCount: q.shape[2], keyCount: k.shape[2])
        let reciprocal = Float(1) / (temperature as! Float)
        hipCheck(dl4s_hip_sdpa_fwd_stats_f32(HIP.context, f(q), f(k), f(v), f(result), f(stats),
                                             Int64(q.shape[0]), Int64(q.shape[1]), Int64(q.shape[2]), Int64(k.shape[2]), Int64(q.shape[3]),
                                             reciprocal, descriptor.kind == Int32(DL4S_MASK_NONE.rawValue) ? nil : &descriptor, attentionFlags))
    }

    public static func fusedAttentionBackward<N: NumericType>(q: ShapedBuffer<N, HIP>, k: ShapedBuffer<N, HIP>, v: ShapedBuffer<N, HIP>,
                                                              mask: ShapedBuffer<N, HIP>?, result: ShapedBuffer<N, HIP>,
                                                              stats: ShapedBuffer<N, HIP>, resultGradient: ShapedBuffer<N, HIP>,
                                                              qGradient: ShapedBuffer<N, HIP>, kGradient: ShapedBuffer<N, HIP>,
                                                              vGradient: ShapedBuffer<N, HIP>, temperature: N) {
        var descriptor = self.descriptor(for: mask, batchSize: q.shape[0], heads: q.shape[1], queryCount: q.shape[2], keyCount: k.shape[2])
        let reciprocal = Float(1) / (temperature as! Float)
        hipCheck(dl4s_hip_sdpa_bwd_f32(HIP.context, f(q), f(k), f(v), f(result), f(stats), f(resultGradient),
                                       f(qGradient), f(kGradient), f(vGradient),
                                       Int64(q.shape[0]), Int64(q.shape[1]), Int64(q.shape[2]), Int64(k.shape[2]), Int64(q.shape[3]),
                                       reciprocal, descriptor.kind == Int32(DL4S_MASK_NONE.rawValue) ? nil : &descriptor, attentionFlags))
    }
}

/// Mask buffers the fused attention calls have looked at (see `HIPEngine.descriptor(for:batchSize:heads:queryCount:keyCount:)`),
/// keyed by the buffer's device address.  An entry owns the device memory of its valid key counts or tile classes.  It is
/// dropped when the buffer it describes is freed (`HIPMemory.free`, which also covers offset views into the freed
/// allocation) or written through `HIPMemory` (`assign`, `set(slice:)`, `setPointee`); the engine's operators always
/// write to result buffers they have just allocated, so nothing else changes a mask under its entry.
enum HIPPreparedMasks {
    struct Entry {
        var descriptor: dl4s_mask_desc
        var shape: [Int]
        var extents: [Int]
        var lengths: UnsafeMutableRawPointer?
        var classes: UnsafeMutableRawPointer?
    }
    static var entries: [UnsafeMutableRawPointer: Entry] = [:]
    static let lock = NSLock()

    static func release(_ entry: Entry) {
        if let lengths = entry.lengths { hipCheck(dl4s_hip_free(HIP.context, lengths)) }
        if let classes = entry.classes { hipCheck(dl4s_hip_free(HIP.context, classes)) }
    }

    static func descriptor<N: NumericType>(for mask: ShapedBuffer<N, HIP>, batchSize: Int, heads: Int, queryCount: Int, keyCount: Int) -> dl4s_mask_desc {
        let key = mask.values.memory.ptr
        let extents = [batchSize, heads, queryCount, keyCount]
        lock.lock()
        defer { lock.unlock() }
        if let known = entries[key], known.shape == mask.shape, known.extents == extents {
            return known.descriptor
        }
        if let stale = entries.removeValue(forKey: key) { release(stale) }
        var dense = HIPEngine.denseDescriptor(for: mask)
        var entry = Entry(descriptor: dense, shape: mask.shape, extents: extents, lengths: nil, classes: nil)
        let (b, h, lq, lk) = (Int64(batchSize), Int64(heads), Int64(queryCount), Int64(keyCount))
        var classBytes = 0
        // a shape that does not fit the problem: the attention call reports it
        guard dl4s_hip_mask_classes_size(&dense, b, h, lq, lk, &classBytes) == 0 else { return dense }
        hipCheck(dl4s_hip_alloc(HIP.context, max(batchSize, 1) * MemoryLayout<Int32>.stride, &entry.lengths))
        var described = dl4s_mask_desc()
        hipCheck(dl4s_hip_mask_describe_f32(HIP.context, &dense, b, h, lq, lk, entry.lengths!.assumingMemoryBound(to: Int32.self), &described))
        if described.kind == Int32(DL4S_MASK_DENSE_F32.rawValue) {
            hipCheck(dl4s_hip_alloc(HIP.context, max(classBytes, 1), &entry.classes))
            hipCheck(dl4s_hip_mask_classify_f32(HIP.context, &dense, b, h, lq, lk, entry.classes!.assumingMemoryBound(to: UInt8.self)))
            described.classes = UnsafePointer(entry.classes!.assumingMemoryBound(to: UInt8.self))
        }
        entry.descriptor = described
        entries[key] = entry
        return described
    }

    /// Drops the entries of mask buffers inside [start, start + bytes): the allocation is being freed or written.
    static func forget(from start: UnsafeMutableRawPointer, bytes: Int) {
        lock.lock()
        defer { lock.unlock() }
        if entries.isEmpty { return }
        let end = start + max(bytes, 1)
        for key in entries.keys.filter({ $0 >= start && $0 < end }) {
            release(entries.removeValue(forKey: key)!)
        }
    }
}

/// The three gradients of one fused attention call, computed together on the first request and handed out one by one
/// (the three closures of a TensorContext are called separately; Tensor/Operators/Stack.swift:104-121 caches its unstack
/// the same way).
final class FusedAttentionGradients<Element: NumericType, Device: DeviceType> {
    var gradients: (q: Tensor<Element, Device>, k: Tensor<Element, Device>, v: Tensor<Element, Device>)?
    var upstream: Tensor<Element, Device>?
}

extension ScaledDotProductAttention {
    /// The fused path of `callAsFunction`: nil when the device's engine has no fused attention, or when gradients are
    /// required and the key and value dims differ (the training form needs them equal).  With gradients required the
    /// result carries a TensorContext whose closures run the fused backward - the mechanism every operator uses, e.g.
    /// Tensor/Operators/Unary.swift:40-53.
    func fusedForward(q: Tensor<Element, Device>, k: Tensor<Element, Device>, v: Tensor<Element, Device>,
                      mask: Tensor<Element, Device>?) -> Tensor<Element, Device>? {
        // outside what the fused call takes - head dims above 256, a mask with more than four axes - and for a mask that
        // requires a gradient (the operator sequence propagates through `mask * 1e9`, the fused call does not) the layer
        // runs its operator sequence
        guard Device.Engine.hasFusedAttention, q.dim == 4, v.dim == 4, q.shape[3] <= 256, v.shape[3] <= 256,
              (mask?.dim ?? 0) <= 4, !(mask?.requiresGradient ?? false) else {
            return nil
        }
        let needsGradient = q.requiresGradient || k.requiresGradient || v.requiresGradient
        if needsGradient && q.shape[3] != v.shape[3] {
            return nil
        }
        let out = Device.Memory.allocateBuffer(withShape: [q.shape[0], q.shape[1], q.shape[2], v.shape[3]], type: Element.self)
        if !needsGradient {
            Device.Engine.fusedAttention(q: q.values, k: k.values, v: v.values, mask: mask?.values, result: out, temperature: temperature)
            return Tensor(using: out, context: nil)
        }
        let stats = Device.Memory.allocateBuffer(withShape: [q.shape[0], q.shape[1], q.shape[2], 2], type: Element.self)
        Device.Engine.fusedAttentionForwardStats(q: q.values, k: k.values, v: v.values, mask: mask?.values, result: out, stats: stats,
                                                 temperature: temperature)
        let result = Tensor<Element, Device>(using: out, context: nil)
        let statistics = Tensor<Element, Device>(using: stats, context: nil)     // owned by the closures below, freed with the graph
        let cache = FusedAttentionGradients<Element, Device>()
        let temperature = self.temperature
        func gradients(_ upstream: Tensor<Element, Device>) -> (q: Tensor<Element, Device>, k: Tensor<Element, Device>, v: Tensor<Element, Device>) {
            if let known = cache.gradients, let seen = cache.upstream, seen.handle === upstream.handle {
                return known
            }
            let dq = Device.Memory.allocateBuffer(withShape: q.shape, type: Element.self)
            let dk = Device.Memory.allocateBuffer(withShape: k.shape, type: Element.self)
            let dv = Device.Memory.allocateBuffer(withShape: v.shape, type: Element.self)
            Device.Engine.fusedAttentionBackward(q: q.values, k: k.values, v: v.values, mask: mask?.values, result: result.values,
                                                 stats: statistics.values, resultGradient: upstream.values, qGradient: dq, kGradient: dk,
                                                 vGradient: dv, temperature: temperature)
            let triple = (q: Tensor<Element, Device>(using: dq, context: nil), k: Tensor<Element, Device>(using: dk, context: nil),
                          v: Tensor<Element, Device>(using: dv, context: nil))
            cache.gradients = triple
            cache.upstream = upstream
            return triple
        }
        // a view of the same storage that carries the context (the buffer is owned by `result`, which the closures keep alive)
        return Tensor(handle: result.handle, shape: result.shape, context: TensorContext(tag: "fusedAttention", sources: [q, k, v], backpropagate: [
            { gradients($0).q }, { gradients($0).k }, { gradients($0).v }
        ]))
    }
}
