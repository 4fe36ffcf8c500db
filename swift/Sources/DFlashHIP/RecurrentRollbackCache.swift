// Rollback caches of the verify loop: Sources/DFlash/RecurrentRollbackCache.swift over the cache handles of
// include/dflash_cache.h.  Same protocol and method names (`DFlashRollbackCache` :12-18,
// `RecurrentRollbackCache` :34-182, `MambaSnapshotCache` :193-232).
//
// How the functional updates of the reference map onto device buffers.  An MLXArray is immutable and
// reference-counted: the verify forward makes `self[1]` a NEW array while the snapshot keeps the old one
// alive (:59-71).  Here the same holds: the forward writes the post-verify state and conv window into new
// arrays and assigns them to the slots (`cache[1] = newState`), the snapshot keeps references to the
// pre-verify arrays.  `rollback` replays the accepted prefix from the snapshot INTO the post-verify arrays
// (their content, the rejected state, is dead), so after it the slots hold the same array objects with the
// rolled-back values; after a snapshot-only restore they hold the pre-verify arrays again.

import CDFlashHIP
import Foundation

// MARK: - DFlashRollbackCache

public protocol DFlashRollbackCache: AnyObject {
    var isArmed: Bool { get }
    func armRollback(prefixLen: Int)
    func rollback(nAccepted: Int)
    func clearTransients()
    func recordTape(tape: MLXArray, k: MLXArray, g: MLXArray, qkv: MLXArray)
}

/// What the shim needs of the model package's `KVCache` protocol (mlx-swift-lm, absent from the reference tree):
/// an offset, trimming, and for recurrent caches two array slots.
public protocol KVCache: AnyObject {
    var offset: Int { get set }
    var isTrimmable: Bool { get }
    @discardableResult func trim(_ n: Int) -> Int
}

/// Stand-in for the model package's `MambaCache`: two array slots (0 = conv window [B, K-1, C], 1 = recurrent
/// state [B, Hv, Dv, Dk]) and the token offset, mirrored into a library handle.
open class MambaCache: KVCache, @unchecked Sendable {
    let handle: OpaquePointer
    private var slots: [MLXArray?] = [nil, nil]

    init(kind: Int32, convKernelSize: Int) {
        guard let h = dflash_cache_create(kind, Int32(convKernelSize)) else {
            DFlashKernels.fail(DFLASH_INVALID, "dflash_cache_create")
        }
        handle = h
    }

    public convenience init() { self.init(kind: DFLASH_CACHE_MAMBA, convKernelSize: 4) }

    deinit { dflash_cache_destroy(handle) }

    public subscript(i: Int) -> MLXArray? {
        get { slots[i] }
        set {
            slots[i] = newValue
            let rc = dflash_cache_set_slot(handle, Int32(i), newValue?.pointer)
            if rc != DFLASH_OK { DFlashKernels.fail(rc, "dflash_cache_set_slot") }
        }
    }

    public var offset: Int {
        get { Int(dflash_cache_offset(handle)) }
        set {
            let rc = dflash_cache_set_offset(handle, Int64(newValue))
            if rc != DFLASH_OK { DFlashKernels.fail(rc, "dflash_cache_set_offset") }
        }
    }

    public var isTrimmable: Bool { true }

    @discardableResult
    open func trim(_ n: Int) -> Int { Int(dflash_cache_trim(handle, Int64(n))) }

    /// After the library has changed the handle's slot pointers (a restore or a rollback), make the Swift-side
    /// slots name the arrays those pointers belong to: the current ones or the snapshot's.
    func adoptSlots(candidates: [MLXArray?]) {
        for i in 0 ..< 2 {
            let p = dflash_cache_get_slot(handle, Int32(i))
            if slots[i]?.pointer == p { continue }
            slots[i] = p == nil ? nil : candidates.compactMap { $0 }.first { $0.pointer == p }
            precondition(p == nil || slots[i] != nil, "cache slot \(i) points at a buffer the shim does not hold")
        }
    }
}

// MARK: - RecurrentRollbackCache

/// `RecurrentRollbackCache` (:34-182): rollback by replaying the innovation tape.
public final class RecurrentRollbackCache: MambaCache, DFlashRollbackCache, @unchecked Sendable {

    /// `RecurrentRollbackCache.defaultConvKernelSize` (:135).
    public nonisolated(unsafe) static var defaultConvKernelSize: Int = 4

    // References that keep the recorded arrays and the snapshot alive until the cycle's rollback or clear.
    private var tape: MLXArray?
    private var tapeK: MLXArray?
    private var tapeG: MLXArray?
    private var tapeQKV: MLXArray?
    private var snapshotState: [MLXArray?]?

    public init(convKernelSize: Int = 4) {
        super.init(kind: DFLASH_CACHE_TAPE, convKernelSize: convKernelSize)
    }

    public var isArmed: Bool { dflash_cache_is_armed(handle) != 0 }

    /// `armRollback(prefixLen:)` (:63-71): arm, drop any old tape, snapshot both slots by reference.
    public func armRollback(prefixLen: Int = 0) {
        tape = nil; tapeK = nil; tapeG = nil; tapeQKV = nil
        snapshotState = [self[0], self[1]]
        let rc = dflash_cache_arm_rollback(handle, Int64(prefixLen))
        if rc != DFLASH_OK { DFlashKernels.fail(rc, "armRollback") }
    }

    /// `recordTape(tape:k:g:qkv:)` (:75-85).  Called by the GatedDelta layer after
    /// `DFlashKernelRegistry.provider!.gatedDeltaKernelWithTape`, and after it has assigned the new state and
    /// conv window to the slots.
    public func recordTape(tape: MLXArray, k: MLXArray, g: MLXArray, qkv: MLXArray) {
        self.tape = tape; self.tapeK = k; self.tapeG = g; self.tapeQKV = qkv
        guard let state = self[1] else { return }
        let rc = dflash_cache_record_tape(
            handle, tape.pointer, DFlashKernels.code(tape, "tape"), k.pointer, g.pointer, DFlashKernels.code(k, "k"),
            Int32(g.ndim), qkv.pointer, Int32(qkv.dtype.size), DFlashKernels.code(state, "state"),
            Int32(k.dim(0)), Int32(k.dim(1)), Int32(k.dim(2)), Int32(tape.dim(2)), Int32(k.dim(3)), Int32(tape.dim(3)),
            Int32(qkv.dim(-1)))
        if rc != DFLASH_OK { DFlashKernels.fail(rc, "recordTape") }
    }

    /// `rollback(nAccepted:)` (:95-131): restore the snapshot, replay `nAccepted + 1` steps (:115), rebuild the
    /// conv window (:139-158), clear.  Enqueued on DFlashStream.current.
    public func rollback(nAccepted: Int) {
        let rc = dflash_cache_rollback(handle, DFlashStream.current.raw, Int32(nAccepted))
        if rc != DFLASH_OK { DFlashKernels.fail(rc, "rollback") }   // the library left the cache armed and untouched
        adoptSlots(candidates: (snapshotState ?? []) + [self[0], self[1]])
        dropReferences()
    }

    /// `clearTransients()` (:163-170).
    public func clearTransients() {
        _ = dflash_cache_clear_transients(handle)
        dropReferences()
    }

    /// Called by `restoreTargetCacheAfterAcceptance` once the library has rolled the whole list back.
    func didRollbackInLibrary() {
        adoptSlots(candidates: (snapshotState ?? []) + [self[0], self[1]])
        dropReferences()
    }

    private func dropReferences() {
        // The replay reads the tape and the snapshot on the stream: the arrays may only be released once that
        // work has run.  DeviceArray frees with hipFree, which waits for the device; a pooling allocator must
        // free in stream order.
        tape = nil; tapeK = nil; tapeG = nil; tapeQKV = nil
        snapshotState = nil
    }

    /// `trim(_:)` (:175-181): only the offset moves; the tape rollback does the rest.
    @discardableResult
    public override func trim(_ n: Int) -> Int { Int(dflash_cache_trim(handle, Int64(n))) }
}

// MARK: - MambaSnapshotCache

/// `MambaSnapshotCache` (:193-232): restores the pre-verify state, no replay.
public final class MambaSnapshotCache: MambaCache, DFlashRollbackCache, @unchecked Sendable {

    private var snapshotConv: MLXArray?
    private var snapshotRecurrent: MLXArray?

    public init() {
        super.init(kind: DFLASH_CACHE_SNAPSHOT, convKernelSize: 4)
    }

    public var isArmed: Bool { dflash_cache_is_armed(handle) != 0 }

    public func armRollback(prefixLen: Int = 0) {
        snapshotConv = self[0]
        snapshotRecurrent = self[1]
        let rc = dflash_cache_arm_rollback(handle, Int64(prefixLen))
        if rc != DFLASH_OK { DFlashKernels.fail(rc, "armRollback") }
    }

    public func rollback(nAccepted: Int) {
        let rc = dflash_cache_rollback(handle, DFlashStream.current.raw, Int32(nAccepted))
        if rc != DFLASH_OK { DFlashKernels.fail(rc, "rollback") }
        didRollbackInLibrary()
    }

    func didRollbackInLibrary() {
        adoptSlots(candidates: [snapshotConv, snapshotRecurrent, self[0], self[1]])
        snapshotConv = nil
        snapshotRecurrent = nil
    }

    public func clearTransients() {
        _ = dflash_cache_clear_transients(handle)
        snapshotConv = nil
        snapshotRecurrent = nil
    }

    public func recordTape(tape: MLXArray, k: MLXArray, g: MLXArray, qkv: MLXArray) {
        // no tape for snapshot-based rollback (:222-224)
    }

    @discardableResult
    public override func trim(_ n: Int) -> Int { Int(dflash_cache_trim(handle, Int64(n))) }
}

/// A trimmable attention cache as the rollback sees it (`KVCacheSimple` lives in the model package): only the
/// offset matters here; rows beyond it are overwritten by the next verify block.
public final class AttentionKVCacheHandle: KVCache, @unchecked Sendable {
    let handle: OpaquePointer
    public init() {
        guard let h = dflash_cache_create(DFLASH_CACHE_KV, 0) else { DFlashKernels.fail(DFLASH_INVALID, "dflash_cache_create") }
        handle = h
    }
    deinit { dflash_cache_destroy(handle) }
    public var offset: Int {
        get { Int(dflash_cache_offset(handle)) }
        set { _ = dflash_cache_set_offset(handle, Int64(newValue)) }
    }
    public var isTrimmable: Bool { true }
    @discardableResult public func trim(_ n: Int) -> Int { Int(dflash_cache_trim(handle, Int64(n))) }
}
