// swift-tools-version:5.9
// DFlashHIP: the Swift face of libdflash_hip.so (gfx950), with the public signatures of SwiftLM's
// `DFlash` target (Sources/DFlash, wired at Package.swift:105-112 of the reference).
//
// Not compiled in this repository's build image (it has no Swift toolchain): these sources are the
// drop-in contract.  To use them inside SwiftLM, add this package as a dependency of the `DFlash`
// target (or copy the two targets below into SwiftLM's Package.swift) and build libdflash_hip.so with
// `make -C swiftlm_amd/csrc`.
import PackageDescription

let package = Package(
    name: "DFlashHIP",
    products: [
        .library(name: "DFlashHIP", targets: ["DFlashHIP"]),
    ],
    targets: [
        // C module: module.modulemap + a one-line umbrella header that includes the two ABI headers of
        // this repository (include/dflash_hip.h, include/dflash_cache.h) and the few HIP runtime calls the
        // shim needs for memory (declared in hip_min.h; they come from libamdhip64).
        .systemLibrary(name: "CDFlashHIP", path: "Sources/CDFlashHIP"),
        .target(
            name: "DFlashHIP",
            dependencies: ["CDFlashHIP"],
            path: "Sources/DFlashHIP",
            linkerSettings: [
                .unsafeFlags(["-L", "../swiftlm_amd/lib", "-L", "/opt/rocm/lib"]),
                .linkedLibrary("dflash_hip"),
                .linkedLibrary("amdhip64"),
            ]
        ),
    ]
)
