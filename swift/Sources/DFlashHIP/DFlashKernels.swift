// DFlashKernels: the static entry points of Sources/DFlash/DFlashKernels.swift over libdflash_hip.so.
//
// Same names, argument labels and result shapes as the reference (tapeReplayKernel :252-258,
// gatedDeltaKernelWithTape :316-324, batchedSDPA2Pass :737-743, sdpaFallback :818-824,
// DFlashKernelsInstance :832-843).  Each call is functional: inputs are never written, results are
// freshly allocated arrays, and the work is enqueued on DFlashStream.current without synchronising.
//
// Where the reference falls back to its ops path (CPU device, DFLASH_FORCE_OPS, a head dim the Metal
// kernels do not take: :259-261, :271-273) this library returns DFLASH_UNSUPPORTED.  There is no
// second implementation inside the shim; a host that has one installs it in `opsFallback`.

import CDFlashHIP
import Foundation

/// The reference's ops implementations (DFlashKernels.swift:371-466), if the host runtime has them.
public struct DFlashOpsFallback: Sendable {
    public var tapeReplay: @Sendable (_ tape: MLXArray, _ k: MLXArray, _ g: MLXArray, _ state: MLXArray, _ mask: MLXArray?) -> MLXArray
    public var gatedDeltaWithTape: @Sendable (_ q: MLXArray, _ k: MLXArray, _ v: MLXArray, _ g: MLXArray, _ beta: MLXArray,
                                              _ state: MLXArray, _ mask: MLXArray?) -> (MLXArray, MLXArray, MLXArray)
    public var sdpa: @Sendable (_ queries: MLXArray, _ keys: MLXArray, _ values: MLXArray, _ scale: Float, _ mask: MLXArray?) -> MLXArray
}

public enum DFlashKernels {

    public static let shared = DFlashKernelsInstance()

    /// Installed by a host that can run the reference's ops path; nil here.
    public nonisolated(unsafe) static var opsFallback: DFlashOpsFallback? = nil

    /// Called when the library reports inconsistent arguments or a HIP failure (the reference has no error
    /// channel on these entry points).  The default stops the process with the library's message.
    public nonisolated(unsafe) static var errorHandler: (DFlashError) -> Never = { fatalError($0.description) }

    static func fail(_ rc: Int32, _ what: String) -> Never {
        errorHandler(DFlashError(status: rc, message: "\(what): " + String(cString: dflash_last_error())))
    }

    static func code(_ a: MLXArray, _ what: String) -> Int32 {
        guard let c = a.dtype.code else { fail(DFLASH_UNSUPPORTED, "\(what): element type \(a.dtype) is not supported") }
        return c
    }

    // MARK: - Tape replay

    /// `tapeReplayKernel(tape:k:g:state:mask:)`, DFlashKernels.swift:252-301.
    /// tape [B,T,Hv,Dv], k [B,T,Hk,Dk], g [B,T,Hv] or [B,T,Hv,Dk], state [B,Hv,Dv,Dk], mask [B,T].
    /// Returns the replayed state, in `state`'s element type.
    public static func tapeReplayKernel(
        tape: MLXArray,
        k: MLXArray,
        g: MLXArray,
        state: MLXArray,
        mask: MLXArray? = nil
    ) -> MLXArray {
        let (B, T, Hk, Dk) = (k.dim(0), k.dim(1), k.dim(2), k.dim(3))
        let (Hv, Dv) = (tape.dim(2), tape.dim(3))
        let out = MLXArray(shape: state.shape, dtype: state.dtype)
        let rc = dflash_tape_replay(
            DFlashStream.current.raw, tape.pointer, code(tape, "tape"), k.pointer, g.pointer, code(k, "k"), Int32(g.ndim),
            state.pointer, out.pointer, code(state, "state"), mask?.pointer, mask.map { code($0, "mask") } ?? 0,
            Int32(B), Int32(T), Int32(Hk), Int32(Hv), Int32(Dk), Int32(Dv))
        if rc == DFLASH_UNSUPPORTED, let ops = opsFallback { return ops.tapeReplay(tape, k, g, state, mask) }
        if rc != DFLASH_OK { fail(rc, "tapeReplayKernel") }
        return out
    }

    // MARK: - GatedDelta forward with tape

    /// `gatedDeltaKernelWithTape(q:k:v:g:beta:state:mask:)`, DFlashKernels.swift:316-367.
    /// Returns (y [B,T,Hv,Dv] in q's type, new state, innovation tape [B,T,Hv,Dv] float32).
    /// The new state keeps `state`'s element type, as the reference's ops path does (:409-466); the
    /// reference's Metal kernel returns it in q's type (:340,:364), so a host that relies on that passes
    /// the state already in q's type (the library then re-rounds it after every step as that kernel does).
    public static func gatedDeltaKernelWithTape(
        q: MLXArray,
        k: MLXArray,
        v: MLXArray,
        g: MLXArray,
        beta: MLXArray,
        state: MLXArray,
        mask: MLXArray? = nil
    ) -> (MLXArray, MLXArray, MLXArray) {
        let (B, T, Hk, Dk) = (k.dim(0), k.dim(1), k.dim(2), k.dim(3))
        let (Hv, Dv) = (v.dim(2), v.dim(3))
        let y = MLXArray(shape: [B, T, Hv, Dv], dtype: q.dtype)
        let tape = MLXArray(shape: [B, T, Hv, Dv], dtype: .float32)
        let out = MLXArray(shape: state.shape, dtype: state.dtype)
        let rc = dflash_gated_delta_tape(
            DFlashStream.current.raw, q.pointer, k.pointer, v.pointer, g.pointer, Int32(g.ndim), beta.pointer, code(q, "q"),
            state.pointer, out.pointer, code(state, "state"), y.pointer, tape.pointer.assumingMemoryBound(to: Float.self),
            mask?.pointer, mask.map { code($0, "mask") } ?? 0,
            Int32(B), Int32(T), Int32(Hk), Int32(Hv), Int32(Dk), Int32(Dv))
        if rc == DFLASH_UNSUPPORTED, let ops = opsFallback { return ops.gatedDeltaWithTape(q, k, v, g, beta, state, mask) }
        if rc != DFLASH_OK { fail(rc, "gatedDeltaKernelWithTape") }
        return (y, out, tape)
    }

    // MARK: - Batched SDPA

    /// `batchedSDPA2Pass(queries:keys:values:scale:mask:)`, DFlashKernels.swift:737-815.
    /// queries [B,Hq,16,D], keys/values [B,Hk,N,D] with N including the 16 block tokens; `mask` is the
    /// optional additive mask [B,Hq,16,N] in the input type.  Returns nil exactly where the reference
    /// does (:744-758): the caller then uses `sdpaFallback`.
    public static func batchedSDPA2Pass(
        queries: MLXArray,
        keys: MLXArray,
        values: MLXArray,
        scale: Float,
        mask: MLXArray? = nil
    ) -> MLXArray? {
        return batchedSDPA2PassWithLSE(queries: queries, keys: keys, values: values, scale: scale, mask: mask, wantLSE: false)?.0
    }

    /// The same call returning the float32 logsumexp [B,Hq,16] as well (no counterpart in the reference).
    public static func batchedSDPA2PassWithLSE(
        queries: MLXArray, keys: MLXArray, values: MLXArray, scale: Float, mask: MLXArray? = nil, wantLSE: Bool = true
    ) -> (MLXArray, MLXArray?)? {
        guard queries.ndim == 4, keys.ndim == 4, values.ndim == 4 else { return nil }
        let (B, Hq, qLen, D) = (queries.dim(0), queries.dim(1), queries.dim(2), queries.dim(3))
        let (Hk, nKV, Vdim) = (keys.dim(1), keys.dim(2), values.dim(3))
        guard qLen == 16 else { return nil }
        guard queries.dtype == .bfloat16 || queries.dtype == .float16 else { return nil }
        guard (D == 128 || D == 256) && D == Vdim else { return nil }
        guard Hk > 0 && Hq % Hk == 0 else { return nil }
        guard keys.dtype == queries.dtype, values.dtype == queries.dtype, values.shape == keys.shape else { return nil }

        let need = dflash_sdpa_workspace_bytes(Int32(B), Int32(Hq), Int32(Hk), Int32(qLen), Int32(nKV), Int32(D))
        guard need > 0 else { return nil }
        let workspace = MLXArray(shape: [need], dtype: .uint8)
        let out = MLXArray(shape: queries.shape, dtype: queries.dtype)
        let lse: MLXArray? = wantLSE ? MLXArray(shape: [B, Hq, qLen], dtype: .float32) : nil
        let dt = code(queries, "queries")
        let rc: Int32
        if let mask = mask {
            // the reference casts the mask to the input type (:783-787); here it must already have it
            guard mask.dtype == queries.dtype, mask.shape == [B, Hq, qLen, nKV] else { return nil }
            rc = dflash_sdpa_block_causal_masked(
                DFlashStream.current.raw, queries.pointer, keys.pointer, values.pointer, mask.pointer, out.pointer,
                lse?.pointer.assumingMemoryBound(to: Float.self), dt, scale,
                Int32(B), Int32(Hq), Int32(Hk), Int32(qLen), Int32(nKV), Int32(D),
                Int64(Hk * nKV * D), Int64(nKV * D), nil, workspace.pointer, need)
        } else {
            rc = dflash_sdpa_block_causal(
                DFlashStream.current.raw, queries.pointer, keys.pointer, values.pointer, out.pointer,
                lse?.pointer.assumingMemoryBound(to: Float.self), dt, scale,
                Int32(B), Int32(Hq), Int32(Hk), Int32(qLen), Int32(nKV), Int32(D),
                Int64(Hk * nKV * D), Int64(nKV * D), nil, workspace.pointer, need)
        }
        if rc == DFLASH_UNSUPPORTED { return nil }
        if rc != DFLASH_OK { fail(rc, "batchedSDPA2Pass") }
        // `workspace` is released when this scope ends; the runtime's allocator must not hand the memory out
        // again before the stream has run the two kernels (hipFree synchronises; a pooling allocator frees
        // in stream order).
        return (out, lse)
    }

    /// `sdpaFallback(queries:keys:values:scale:mask:)`, DFlashKernels.swift:818-828: the array library's
    /// general attention.  This package ships only the verify-block kernel, so shapes it does not cover
    /// go to the host's installed fallback or are an error.
    public static func sdpaFallback(
        queries: MLXArray,
        keys: MLXArray,
        values: MLXArray,
        scale: Float,
        mask: MLXArray? = nil
    ) -> MLXArray {
        if let out = batchedSDPA2Pass(queries: queries, keys: keys, values: values, scale: scale, mask: mask) { return out }
        if let ops = opsFallback { return ops.sdpa(queries, keys, values, scale, mask) }
        fail(DFLASH_UNSUPPORTED, "sdpaFallback: shape or type outside the verify-block attention kernel and no fallback installed")
    }
}

/// `DFlashKernelsInstance`, DFlashKernels.swift:832-843.
public final class DFlashKernelsInstance: DFlashKernelProvider, @unchecked Sendable {
    public init() {}
    public func gatedDeltaKernelWithTape(
        q: MLXArray, k: MLXArray, v: MLXArray,
        g: MLXArray, beta: MLXArray,
        state: MLXArray, mask: MLXArray?
    ) -> (MLXArray, MLXArray, MLXArray) {
        DFlashKernels.gatedDeltaKernelWithTape(
            q: q, k: k, v: v, g: g, beta: beta,
            state: state, mask: mask
        )
    }
}
