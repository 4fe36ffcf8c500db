// The verify loop's device-side pieces: Sources/DFlash/DFlashRuntime.swift
// (`buildSuppressTokenMask` :105-115, `greedyTokensWithMask` :118-128, `matchAcceptanceLength` :133-142,
// `restoreTargetCacheAfterAcceptance` :188-223) over libdflash_hip.so.  The generation loop itself
// (`generateStreaming`, :308-634) stays the reference's: it calls these.

import CDFlashHIP
import Foundation

public enum DFlashRuntime {

    // MARK: - Token Utilities

    /// `buildSuppressTokenMask(vocabSize:suppressTokenIDs:)` (:105-115): uint8 [vocab], 1 = suppressed.
    public static func buildSuppressTokenMask(
        vocabSize: Int,
        suppressTokenIDs: [Int]?
    ) -> MLXArray? {
        let ids = Set((suppressTokenIDs ?? []).filter { $0 >= 0 && $0 < vocabSize })
        guard !ids.isEmpty else { return nil }
        var mask = [UInt8](repeating: 0, count: vocabSize)
        for id in ids { mask[id] = 1 }
        return MLXArray(mask, shape: [vocabSize], dtype: .uint8)
    }

    /// `greedyTokensWithMask(logits:suppressTokenMask:)` (:118-128): argmax over the last axis of [T, vocab]
    /// logits with suppressed tokens floored at -1e9; uint32 tokens, lowest index on ties.
    public static func greedyTokensWithMask(
        logits: MLXArray,
        suppressTokenMask: MLXArray? = nil
    ) -> MLXArray {
        let (T, V) = (logits.dim(-2), logits.dim(-1))
        let tokens = MLXArray(shape: [T], dtype: .uint32)
        let need = dflash_greedy_workspace_bytes(Int32(T), Int32(V))
        let ws = MLXArray(shape: [need], dtype: .uint8)
        let rc = dflash_greedy_tokens_with_mask(
            DFlashStream.current.raw, logits.pointer, DFlashKernels.code(logits, "logits"), Int32(T), Int32(V),
            suppressTokenMask?.pointer.assumingMemoryBound(to: UInt8.self),
            tokens.pointer.assumingMemoryBound(to: UInt32.self), ws.pointer, need)
        if rc != DFLASH_OK { DFlashKernels.fail(rc, "greedyTokensWithMask") }
        return tokens
    }

    /// `matchAcceptanceLength(draftedTokens:posteriorTokens:)` (:133-142): the number of leading positions at
    /// which the two uint32 token arrays agree, as an int32 scalar on the device (0 for empty input).
    public static func matchAcceptanceLength(
        draftedTokens: MLXArray,
        posteriorTokens: MLXArray
    ) -> MLXArray {
        let count = draftedTokens.dim(0)
        guard count > 0 else { return MLXArray([Int32(0)], shape: [], dtype: .int32) }
        let out = MLXArray(shape: [], dtype: .int32)
        let rc = dflash_match_acceptance_length(
            DFlashStream.current.raw, draftedTokens.pointer.assumingMemoryBound(to: UInt32.self),
            posteriorTokens.pointer.assumingMemoryBound(to: UInt32.self), Int32(count),
            out.pointer.assumingMemoryBound(to: Int32.self))
        if rc != DFLASH_OK { DFlashKernels.fail(rc, "matchAcceptanceLength") }
        return out
    }

    /// The cycle's integer bookkeeping in one launch and one 16-byte read-back (:490-493, :525-547, :571):
    /// (acceptanceLen, commitCount, stagedFirstNext, start + commitCount).  No counterpart as a single call in
    /// the reference, which does `.item()` on a lazy graph.
    public static func acceptCommit(verifyTokenIDs: MLXArray, posterior: MLXArray, start: Int) -> (Int, Int, Int, Int) {
        let out = MLXArray(shape: [4], dtype: .int32)
        let st = MLXArray([Int32(start)], shape: [1], dtype: .int32)
        let rc = dflash_accept_commit(
            DFlashStream.current.raw, verifyTokenIDs.pointer.assumingMemoryBound(to: UInt32.self),
            posterior.pointer.assumingMemoryBound(to: UInt32.self), Int32(verifyTokenIDs.dim(0)),
            st.pointer.assumingMemoryBound(to: Int32.self), out.pointer.assumingMemoryBound(to: Int32.self))
        if rc != DFLASH_OK { DFlashKernels.fail(rc, "acceptCommit") }
        let v = out.toHost(Int32.self)
        return (Int(v[0]), Int(v[1]), Int(v[2]), Int(v[3]))
    }

    // MARK: - Target Cache Management

    /// `restoreTargetCacheAfterAcceptance(_:targetLen:acceptanceLength:draftedTokens:)` (:188-223).
    /// Fully accepted: rollback caches only clear their transients.  Otherwise tape caches are rolled back (all
    /// caches that share a shape replay in ONE launch), snapshot caches restore, plain Mamba caches take
    /// `offset = targetLen`, trimmable caches are trimmed to `targetLen`.  Returns the nanoseconds spent.
    /// Caches the library does not know (a host cache type that is not one of this file's classes) are handled
    /// here exactly as the reference does.
    @discardableResult
    public static func restoreTargetCacheAfterAcceptance(
        _ cacheEntries: [KVCache],
        targetLen: Int,
        acceptanceLength: Int,
        draftedTokens: Int
    ) -> Int {
        var handles: [OpaquePointer?] = []
        var foreign: [KVCache] = []
        for cache in cacheEntries {
            if let c = cache as? MambaCache { handles.append(c.handle) }
            else if let c = cache as? AttentionKVCacheHandle { handles.append(c.handle) }
            else { foreign.append(cache) }
        }
        var ns: Int64 = 0
        let rc = handles.withUnsafeBufferPointer {
            dflash_restore_target_cache_after_acceptance(
                $0.baseAddress, Int32(handles.count), DFlashStream.current.raw, Int64(targetLen),
                Int32(acceptanceLength), Int32(draftedTokens), &ns)
        }
        // On failure the library has touched nothing: every cache is still armed.
        if rc != DFLASH_OK { DFlashKernels.fail(rc, "restoreTargetCacheAfterAcceptance") }
        let fullyAccepted = draftedTokens > 0 && acceptanceLength == draftedTokens
        for cache in cacheEntries {
            if fullyAccepted {
                (cache as? DFlashRollbackCache)?.clearTransients()
            } else if let c = cache as? RecurrentRollbackCache {
                c.didRollbackInLibrary()
            } else if let c = cache as? MambaSnapshotCache {
                c.didRollbackInLibrary()
            }
        }
        var extraNs = 0
        for cache in foreign {
            if let rollbackCache = cache as? DFlashRollbackCache {
                if fullyAccepted { rollbackCache.clearTransients(); continue }
                let t0 = DispatchTime.now().uptimeNanoseconds
                rollbackCache.rollback(nAccepted: acceptanceLength)
                extraNs += Int(DispatchTime.now().uptimeNanoseconds - t0)
            } else if cache.isTrimmable, cache.offset > targetLen {
                cache.trim(cache.offset - targetLen)
            }
        }
        return Int(ns) + extraNs
    }
}
