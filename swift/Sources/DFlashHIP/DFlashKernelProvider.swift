// `DFlashKernelProvider` / `DFlashKernelRegistry`, Sources/DFlash/DFlashKernelProvider.swift:8-19:
// the hook through which the GatedDelta layer (in the model package) reaches the tape-recording
// forward without a module cycle.  The server sets `DFlashKernelRegistry.provider = DFlashKernels.shared`
// (Sources/SwiftLM/Server.swift:684).

import Foundation

public protocol DFlashKernelProvider: Sendable {
    func gatedDeltaKernelWithTape(
        q: MLXArray, k: MLXArray, v: MLXArray,
        g: MLXArray, beta: MLXArray,
        state: MLXArray, mask: MLXArray?
    ) -> (MLXArray, MLXArray, MLXArray)
}

public struct DFlashKernelRegistry: Sendable {
    public nonisolated(unsafe) static var provider: DFlashKernelProvider? = nil
}
