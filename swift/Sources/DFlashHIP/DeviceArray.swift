// DeviceArray: the tensor type of the shim.
//
// SwiftLM's DFlash sources are written against MLXArray (mlx-swift), which has no ROCm backend; the
// kernels of libdflash_hip.so need nothing from an array but its device pointer, shape and element
// type.  DeviceArray is exactly that, reference-counted like an MLXArray, so that "snapshot by
// reference" (RecurrentRollbackCache.swift:59-71) means the same thing here.  Inside this module
// `MLXArray` is an alias of it, which keeps every public signature identical to the reference's.
// A host runtime with its own tensor type bridges by constructing a DeviceArray over memory it owns
// (`init(borrowing:...)`).

import CDFlashHIP
import Foundation

public enum DType: Sendable {
    case float32, bfloat16, float16, uint8, int32, uint32

    public var size: Int {
        switch self {
        case .float32, .int32, .uint32: return 4
        case .bfloat16, .float16: return 2
        case .uint8: return 1
        }
    }

    /// Element code of include/dflash_hip.h, or nil for types the kernels do not take as data.
    var code: Int32? {
        switch self {
        case .float32: return DFLASH_F32
        case .bfloat16: return DFLASH_BF16
        case .float16: return DFLASH_F16
        case .uint8: return DFLASH_U8
        default: return nil
        }
    }
}

/// Failure of a library call: the status code and the text of dflash_last_error().
public struct DFlashError: Error, CustomStringConvertible {
    public let status: Int32
    public let message: String
    public var description: String { "DFlash (status \(status)): \(message)" }
}

/// Streams are passed through as opaque hipStream_t values; nil is the default stream.
public struct DFlashStream: @unchecked Sendable {
    public var raw: UnsafeMutableRawPointer?
    public init(_ raw: UnsafeMutableRawPointer? = nil) { self.raw = raw }
    /// The stream the static entry points of DFlashKernels enqueue on.
    public nonisolated(unsafe) static var current = DFlashStream()
}

public final class DeviceArray: @unchecked Sendable {
    public let pointer: UnsafeMutableRawPointer
    public let shape: [Int]
    public let dtype: DType
    private let owned: Bool
    /// Keeps the storage of a view alive.
    private let parent: DeviceArray?

    public var ndim: Int { shape.count }
    public var count: Int { shape.reduce(1, *) }
    public var nbytes: Int { count * dtype.size }
    public func dim(_ i: Int) -> Int { shape[i >= 0 ? i : shape.count + i] }

    /// Allocates uninitialised device memory.
    public init(shape: [Int], dtype: DType) {
        var p: UnsafeMutableRawPointer?
        let bytes = max(shape.reduce(1, *) * dtype.size, 1)
        let rc = hipMalloc(&p, bytes)
        precondition(rc == 0 && p != nil, "hipMalloc(\(bytes)) failed: \(String(cString: hipGetErrorString(rc)))")
        self.pointer = p!
        self.shape = shape
        self.dtype = dtype
        self.owned = true
        self.parent = nil
    }

    /// Wraps memory owned by the caller's runtime; it must outlive the array.
    public init(borrowing pointer: UnsafeMutableRawPointer, shape: [Int], dtype: DType) {
        self.pointer = pointer
        self.shape = shape
        self.dtype = dtype
        self.owned = false
        self.parent = nil
    }

    private init(viewOf parent: DeviceArray, byteOffset: Int, shape: [Int]) {
        self.pointer = parent.pointer + byteOffset
        self.shape = shape
        self.dtype = parent.dtype
        self.owned = false
        self.parent = parent
    }

    deinit {
        if owned { _ = hipFree(pointer) }
    }

    /// Zero-filled array (enqueued on the current stream).
    public static func zeros(_ shape: [Int], dtype: DType) -> DeviceArray {
        let a = DeviceArray(shape: shape, dtype: dtype)
        _ = hipMemsetAsync(a.pointer, 0, a.nbytes, DFlashStream.current.raw)
        return a
    }

    /// Host values to the device (synchronous).
    public convenience init<T>(_ values: [T], shape: [Int], dtype: DType) {
        self.init(shape: shape, dtype: dtype)
        precondition(values.count * MemoryLayout<T>.stride == nbytes, "host buffer does not match shape and dtype")
        values.withUnsafeBytes { _ = hipMemcpy(pointer, $0.baseAddress, nbytes, 1) }
    }

    /// Device values to the host, after the current stream has drained.
    public func toHost<T>(_ type: T.Type) -> [T] {
        _ = hipStreamSynchronize(DFlashStream.current.raw)
        var out = [T](unsafeUninitializedCapacity: nbytes / MemoryLayout<T>.stride) { _, n in n = self.nbytes / MemoryLayout<T>.stride }
        out.withUnsafeMutableBytes { _ = hipMemcpy($0.baseAddress, pointer, nbytes, 2) }
        return out
    }

    /// The first `n` entries along axis 1 of a contiguous [B, T, ...] array.  A view when B == 1 (the
    /// verify loop's case: the prefix of a contiguous array is contiguous); otherwise nil, and the
    /// caller passes the full array with an explicit step count instead.
    public func prefixAlongAxis1(_ n: Int) -> DeviceArray? {
        guard ndim >= 2, dim(0) == 1, n <= dim(1) else { return nil }
        var s = shape
        s[1] = n
        return DeviceArray(viewOf: self, byteOffset: 0, shape: s)
    }
}

/// Inside this module the reference's array type name stands for DeviceArray.
public typealias MLXArray = DeviceArray

@inline(__always)
func check(_ rc: Int32, _ what: String) throws {
    if rc != DFLASH_OK {
        throw DFlashError(status: rc, message: "\(what): " + String(cString: dflash_last_error()))
    }
}
