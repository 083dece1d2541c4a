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
    /// broadcast (Util.swift:40-45).  The library classifies the mask's 32 x 32 tiles once per call and reads mask values
    /// only in tiles that are neither all zeros nor all ones, so the masks of TransformerUtil.swift:29-50 cost about what a
    /// structured descriptor costs.
    static func descriptor<N: NumericType>(for mask: ShapedBuffer<N, HIP>?) -> dl4s_mask_desc {
        var descriptor = dl4s_mask_desc()
        guard let mask = mask else {
            descriptor.kind = Int32(DL4S_MASK_NONE.rawValue)
            return descriptor
        }
        precondition(mask.dim <= 4, "attention masks have at most 4 axes")
        let padded = [Int](repeating: 1, count: 4 - mask.dim) + mask.shape
        descriptor.kind = Int32(DL4S_MASK_DENSE_F32.rawValue)
        descriptor.dense = UnsafePointer(f(mask))
        descriptor.shape = (Int64(padded[0]), Int64(padded[1]), Int64(padded[2]), Int64(padded[3]))
        return descriptor
    }

    static var attentionFlags: UInt32 {
        return HIP.strictMasks ? DL4S_SDPA_STRICT : 0
    }

    public static func fusedAttention<N: NumericType>(q: ShapedBuffer<N, HIP>, k: ShapedBuffer<N, HIP>, v: ShapedBuffer<N, HIP>,
                                                      mask: ShapedBuffer<N, HIP>?, result: ShapedBuffer<N, HIP>, temperature: N) {
        precondition(q.dim == 4 && k.dim == 4 && v.dim == 4)
        var descriptor = self.descriptor(for: mask)
        // the reference forms the reciprocal once in Float and multiplies (Engine/CPU/CPUEngine.swift:635)
        let reciprocal = Float(1) / (temperature as! Float)
        hipCheck(dl4s_hip_sdpa_fwd_f32(HIP.context, f(q), f(k), f(v), f(result),
                                       Int64(q.shape[0]), Int64(q.shape[1]), Int64(q.shape[2]), Int64(k.shape[2]),
                                       Int64(q.shape[3]), Int64(v.shape[3]), reciprocal, mask == nil ? nil : &descriptor, attentionFlags))
    }

    public static func fusedAttentionForwardStats<N: NumericType>(q: ShapedBuffer<N, HIP>, k: ShapedBuffer<N, HIP>, v: ShapedBuffer<N, HIP>,
                                                                  mask: ShapedBuffer<N, HIP>?, result: ShapedBuffer<N, HIP>,
                                                                  stats: ShapedBuffer<N, HIP>, temperature: N) {
        precondition(q.dim == 4 && k.dim == 4 && v.dim == 4 && q.shape[3] == v.shape[3], "the training form needs keyDim == valueDim")
        var descriptor = self.descriptor(for: mask)
        let reciprocal = Float(1) / (temperature as! Float)
        hipCheck(dl4s_hip_sdpa_fwd_stats_f32(HIP.context, f(q), f(k), f(v), f(result), f(stats),
                                             Int64(q.shape[0]), Int64(q.shape[1]), Int64(q.shape[2]), Int64(k.shape[2]), Int64(q.shape[3]),
                                             reciprocal, mask == nil ? nil : &descriptor, attentionFlags))
    }

    public static func fusedAttentionBackward<N: NumericType>(q: ShapedBuffer<N, HIP>, k: ShapedBuffer<N, HIP>, v: ShapedBuffer<N, HIP>,
                                                              mask: ShapedBuffer<N, HIP>?, result: ShapedBuffer<N, HIP>,
                                                              stats: ShapedBuffer<N, HIP>, resultGradient: ShapedBuffer<N, HIP>,
                                                              qGradient: ShapedBuffer<N, HIP>, kGradient: ShapedBuffer<N, HIP>,
                                                              vGradient: ShapedBuffer<N, HIP>, temperature: N) {
        var descriptor = self.descriptor(for: mask)
        let reciprocal = Float(1) / (temperature as! Float)
        hipCheck(dl4s_hip_sdpa_bwd_f32(HIP.context, f(q), f(k), f(v), f(result), f(stats), f(resultGradient),
                                       f(qGradient), f(kGradient), f(vGradient),
                                       Int64(q.shape[0]), Int64(q.shape[1]), Int64(q.shape[2]), Int64(k.shape[2]), Int64(q.shape[3]),
                                       reciprocal, mask == nil ? nil : &descriptor, attentionFlags))
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
        guard Device.Engine.hasFusedAttention, q.dim == 4, v.dim == 4 else {
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
