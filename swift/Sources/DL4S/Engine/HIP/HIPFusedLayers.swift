//
//  HIPFusedLayers.swift
//  DL4S
//
//  The forward pass of MultiHeadAttention and PointwiseFeedForward through the library's fused layer forms:
//
//    MultiHeadAttention.callAsFunction (NN/Models/Transformer/MultiHeadAttention.swift:97-127)
//      three projections            one grouped launch                            dl4s_hip_gemm_grouped_f32
//      four permuted(to:) copies    none: the attention call reads and writes the projections' own layout
//                                                                                 dl4s_hip_sdpa_fwd_f32 + DL4S_SDPA_TOKEN_MAJOR
//      fc product, + res, norm      one call, the LayerNorm sums from the product's epilogue
//                                                                                 dl4s_hip_dense_layernorm_f32
//    PointwiseFeedForward.callAsFunction (NN/Models/Transformer/PointwiseFeedForward.swift:67-82)
//      dense1, + bias, GeLU         one call                                      dl4s_hip_dense_fused_f32
//      dense2, + bias, + inputs     one call                                      dl4s_hip_dense_fused_f32
//      norm                         one call                                      dl4s_hip_layernorm_f32
//
//  These forms compute the forward pass only: their results carry no TensorContext, so no gradient flows through a layer
//  that took them.  They are therefore opt-in: `HIP.fusedLayers = true` is the caller's statement that the model runs
//  without gradients (inference, evaluation, decoding); with the default (false) the layers run their operator
//  sequences, with the fused attention hook of HIPFusedAttention.swift - which does supply gradients - inside
//  ScaledDotProductAttention.
//
//  patches/Engine.swift.patch declares the six requirements below in EngineType, patches/MultiHeadAttention.swift.patch
//  and patches/PointwiseFeedForward.swift.patch add the calls of `fusedForward` to the two layers.  The C++ host layer
//  (dl4s_amd/host/dl4s_host.hpp, mode "fused") makes exactly these calls and is what the tests and the benchmark run.
//

import Foundation
import CDL4SHIP

extension EngineType {
    public static var hasFusedLayers: Bool { return false }

    public static func gemmGrouped<N: NumericType>(lhs: [ShapedBuffer<N, Device>], rhs: [ShapedBuffer<N, Device>], results: [ShapedBuffer<N, Device>]) {
        fatalError("\(#function) is not available for \(self)")
    }

    public static func fusedAttentionTokenMajor<N: NumericType>(q: ShapedBuffer<N, Device>, k: ShapedBuffer<N, Device>, v: ShapedBuffer<N, Device>,
                                                                mask: ShapedBuffer<N, Device>?, result: ShapedBuffer<N, Device>, temperature: N) {
        fatalError("\(#function) is not available for \(self)")
    }

    public static func denseFused<N: NumericType>(input: ShapedBuffer<N, Device>, weights: ShapedBuffer<N, Device>, bias: ShapedBuffer<N, Device>?,
                                                  gaussianErrorLinear: Bool, residual: ShapedBuffer<N, Device>?, result: ShapedBuffer<N, Device>) {
        fatalError("\(#function) is not available for \(self)")
    }

    public static func denseLayerNorm<N: NumericType>(input: ShapedBuffer<N, Device>, weights: ShapedBuffer<N, Device>, residual: ShapedBuffer<N, Device>?,
                                                      itemRows: Int, scale: ShapedBuffer<N, Device>, shift: ShapedBuffer<N, Device>,
                                                      result: ShapedBuffer<N, Device>) {
        fatalError("\(#function) is not available for \(self)")
    }

    public static func layerNorm<N: NumericType>(input: ShapedBuffer<N, Device>, itemRows: Int, scale: ShapedBuffer<N, Device>,
                                                 shift: ShapedBuffer<N, Device>, result: ShapedBuffer<N, Device>) {
        fatalError("\(#function) is not available for \(self)")
    }
}

extension HIP {
    /// Whether MultiHeadAttention and PointwiseFeedForward run their forward pass through the fused layer forms.  Their
    /// results carry no gradient context: set it for inference only.  With `strictMasks` the LayerNorm sums are added in
    /// the reference's sequential order as well (dl4s_hip_layernorm_reference_order_f32).
    public static var fusedLayers = false
}

extension HIPEngine {
    public static var hasFusedLayers: Bool { return HIP.fusedLayers }

    public static func gemmGrouped<N: NumericType>(lhs: [ShapedBuffer<N, HIP>], rhs: [ShapedBuffer<N, HIP>], results: [ShapedBuffer<N, HIP>]) {
        precondition(lhs.count == rhs.count && lhs.count == results.count && (1 ... 4).contains(lhs.count), "a group holds one to four products")
        precondition(lhs.allSatisfy { $0.dim == 2 && $0.shape == lhs[0].shape } && rhs.allSatisfy { $0.dim == 2 && $0.shape == rhs[0].shape } &&
                     lhs[0].shape[1] == rhs[0].shape[0], "Matmul operands must have matching shapes")
        var a: [UnsafePointer<Float>?] = lhs.map { UnsafePointer(f($0)) }
        var b: [UnsafePointer<Float>?] = rhs.map { UnsafePointer(f($0)) }
        var c: [UnsafeMutablePointer<Float>?] = results.map { f($0) }
        hipCheck(dl4s_hip_gemm_grouped_f32(HIP.context, Int32(lhs.count), &a, Int64(lhs[0].shape[0]), Int64(lhs[0].shape[1]),
                                           &b, Int64(rhs[0].shape[0]), Int64(rhs[0].shape[1]), &c, 1, 0, 0, 0))
    }

    public static func fusedAttentionTokenMajor<N: NumericType>(q: ShapedBuffer<N, HIP>, k: ShapedBuffer<N, HIP>, v: ShapedBuffer<N, HIP>,
                                                                mask: ShapedBuffer<N, HIP>?, result: ShapedBuffer<N, HIP>, temperature: N) {
        precondition(q.dim == 4 && k.dim == 4 && v.dim == 4 && q.shape[3] == v.shape[3], "the token-major form needs keyDim == valueDim")
        // [batch, length, heads, dim]: heads on axis 2
        var descriptor = self.descriptor(for: mask, batchSize: q.shape[0], heads: q.shape[2], queryCount: q.shape[1], keyCount: k.shape[1])
        let reciprocal = Float(1) / (temperature as! Float)
        hipCheck(dl4s_hip_sdpa_fwd_f32(HIP.context, f(q), f(k), f(v), f(result),
                                       Int64(q.shape[0]), Int64(q.shape[2]), Int64(q.shape[1]), Int64(k.shape[1]),
                                       Int64(q.shape[3]), Int64(v.shape[3]), reciprocal,
                                       descriptor.kind == Int32(DL4S_MASK_NONE.rawValue) ? nil : &descriptor,
                                       attentionFlags | DL4S_SDPA_TOKEN_MAJOR))
    }

    public static func denseFused<N: NumericType>(input: ShapedBuffer<N, HIP>, weights: ShapedBuffer<N, HIP>, bias: ShapedBuffer<N, HIP>?,
                                                  gaussianErrorLinear: Bool, residual: ShapedBuffer<N, HIP>?, result: ShapedBuffer<N, HIP>) {
        precondition(input.dim == 2 && weights.dim == 2 && input.shape[1] == weights.shape[0], "Matmul operands must have matching shapes")
        hipCheck(dl4s_hip_dense_fused_f32(HIP.context, f(input), Int64(input.shape[0]), Int64(input.shape[1]), f(weights), Int64(weights.shape[1]),
                                          bias.map { UnsafePointer(f($0)) }, gaussianErrorLinear ? DL4S_ACT_GELU : DL4S_ACT_NONE,
                                          residual.map { UnsafePointer(f($0)) }, f(result)))
    }

    public static func denseLayerNorm<N: NumericType>(input: ShapedBuffer<N, HIP>, weights: ShapedBuffer<N, HIP>, residual: ShapedBuffer<N, HIP>?,
                                                      itemRows: Int, scale: ShapedBuffer<N, HIP>, shift: ShapedBuffer<N, HIP>,
                                                      result: ShapedBuffer<N, HIP>) {
        precondition(input.dim == 2 && weights.dim == 2 && input.shape[1] == weights.shape[0] && input.shape[0] % itemRows == 0,
                     "Matmul operands must have matching shapes")
        if HIP.strictMasks {
            // the product with its residual, then the statistics in the order the reference adds them
            denseFused(input: input, weights: weights, bias: nil, gaussianErrorLinear: false, residual: residual, result: result)
            layerNorm(input: result, itemRows: itemRows, scale: scale, shift: shift, result: result)
            return
        }
        hipCheck(dl4s_hip_dense_layernorm_f32(HIP.context, f(input), Int64(input.shape[0]), Int64(input.shape[1]), f(weights),
                                              Int64(weights.shape[1]), nil, DL4S_ACT_NONE, residual.map { UnsafePointer(f($0)) },
                                              Int64(itemRows), f(scale), f(shift), f(result)))
    }

    public static func layerNorm<N: NumericType>(input: ShapedBuffer<N, HIP>, itemRows: Int, scale: ShapedBuffer<N, HIP>,
                                                 shift: ShapedBuffer<N, HIP>, result: ShapedBuffer<N, HIP>) {
        precondition(input.dim == 2 && input.shape[0] % itemRows == 0 && scale.shape.reduce(1, *) == input.shape[1] &&
                     shift.shape.reduce(1, *) == input.shape[1], "LayerNorm operands must have matching shapes")
        let items = Int64(input.shape[0] / itemRows)
        if HIP.strictMasks {
            hipCheck(dl4s_hip_layernorm_reference_order_f32(HIP.context, f(input), nil, f(scale), f(shift), f(result),
                                                            items, Int64(itemRows), Int64(input.shape[1])))
        } else {
            hipCheck(dl4s_hip_layernorm_f32(HIP.context, f(input), nil, f(scale), f(shift), f(result),
                                            items, Int64(itemRows), Int64(input.shape[1])))
        }
    }
}

extension MultiHeadAttention {
    /// The fused forward pass of `callAsFunction`, or nil when the device's engine has no fused layer forms or the layer is
    /// outside what they take (active dropout, key and value dims that differ, are no multiple of 4 or exceed 256, keys
    /// and values of different counts): the caller then runs the operator sequence.
    func fusedForward(q: Tensor<Element, Device>, k: Tensor<Element, Device>, v: Tensor<Element, Device>,
                      mask: Tensor<Element, Device>?) -> Tensor<Element, Device>? {
        guard Device.Engine.hasFusedLayers, !dropout.isActive, keyDim == valueDim, keyDim % 4 == 0, keyDim <= 256,
              q.dim == 3, k.dim == 3, v.dim == 3, k.shape[1] == v.shape[1], (mask?.dim ?? 0) <= 4 else {
            return nil
        }
        let batchSize = q.shape[0], queryCount = q.shape[1], keyCount = k.shape[1]
        func projection(_ count: Int) -> ShapedBuffer<Element, Device> {
            return Device.Memory.allocateBuffer(withShape: [batchSize, count, heads, keyDim], type: Element.self)
        }
        func rows(_ t: Tensor<Element, Device>) -> ShapedBuffer<Element, Device> {      // [batch, length, hidden] as [batch * length, hidden]
            return t.values.reshaped(to: [t.shape[0] * t.shape[1], t.shape[2]])
        }
        func flat(_ b: ShapedBuffer<Element, Device>) -> ShapedBuffer<Element, Device> {  // [batch, length, heads, dim] as [batch * length, heads * dim]
            return b.reshaped(to: [b.shape[0] * b.shape[1], b.shape[2] * b.shape[3]])
        }
        // the three projections (MultiHeadAttention.swift:109-111) as one launch when their inputs have one length,
        // keys and values as one launch and the queries by themselves otherwise
        let qp = projection(queryCount), kp = projection(keyCount), vp = projection(keyCount)
        if queryCount == keyCount {
            Device.Engine.gemmGrouped(lhs: [rows(q), rows(k), rows(v)], rhs: [qDense.values, kDense.values, vDense.values],
                                      results: [flat(qp), flat(kp), flat(vp)])
        } else {
            Device.Engine.gemmGrouped(lhs: [rows(k), rows(v)], rhs: [kDense.values, vDense.values], results: [flat(kp), flat(vp)])
            Device.Engine.gemm(lhs: rows(q), rhs: qDense.values, result: flat(qp), alpha: 1.0, beta: 0.0, transposeFirst: false, transposeSecond: false)
        }
        // attention on the projections where the products wrote them; the output lands as [batch, queries, heads * dim]
        // (the four permutations of MultiHeadAttention.swift:113-119 are not made)
        let attended = projection(queryCount)
        Device.Engine.fusedAttentionTokenMajor(q: qp, k: kp, v: vp, mask: mask?.values, result: attended, temperature: attn.temperature)
        Device.Memory.free(qp)
        Device.Memory.free(kp)
        Device.Memory.free(vp)
        // fc, + res and the joint (length, hidden) normalisation of MultiHeadAttention.swift:121-124 in one call
        let out = Device.Memory.allocateBuffer(withShape: [batchSize * queryCount, hiddenDim], type: Element.self)
        Device.Engine.denseLayerNorm(input: flat(attended), weights: fc.values, residual: rows(q), itemRows: queryCount,
                                     scale: norm.scale.values, shift: norm.shift.values, result: out)
        Device.Memory.free(attended)
        return Tensor(using: out.reshaped(to: [batchSize, queryCount, hiddenDim]), context: nil)
    }
}

extension PointwiseFeedForward {
    /// The fused forward pass on `denseInputs` [batchSize * seqlen, size] (PointwiseFeedForward.swift:74-79), or nil when
    /// the device's engine has no fused layer forms or dropout is active.
    func fusedForward(_ denseInputs: Tensor<Element, Device>) -> Tensor<Element, Device>? {
        guard Device.Engine.hasFusedLayers, !dropout.isActive, denseInputs.dim == 2 else {
            return nil
        }
        let rows = denseInputs.shape[0]
        let hidden = Device.Memory.allocateBuffer(withShape: [rows, dense1.weights.shape[1]], type: Element.self)
        Device.Engine.denseFused(input: denseInputs.values, weights: dense1.weights.values, bias: dense1.bias.values,
                                 gaussianErrorLinear: true, residual: nil, result: hidden)
        let sum = Device.Memory.allocateBuffer(withShape: [rows, dense2.weights.shape[1]], type: Element.self)
        Device.Engine.denseFused(input: hidden, weights: dense2.weights.values, bias: dense2.bias.values,
                                 gaussianErrorLinear: false, residual: denseInputs.values, result: sum)
        Device.Memory.free(hidden)
        // every token by itself: the tensor is [batch * length, size] here, so LayerNorm's axes 1..<dim are the features
        let out = Device.Memory.allocateBuffer(withShape: sum.shape, type: Element.self)
        Device.Engine.layerNorm(input: sum, itemRows: 1, scale: norm.scale.values, shift: norm.shift.values, result: out)
        Device.Memory.free(sum)
        return Tensor(using: out, context: nil)
    }
}
