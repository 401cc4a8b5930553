// swift-tools-version: 6.0
// UNCOMPILED: no Swift toolchain exists in the image this library is built in.
// Linux/ROCm package that puts libespresso_hip.so behind a Swift module, in the place the reference gives its
// ANEInterop C target (reference Package.swift:27-41).
import PackageDescription

let package = Package(
    name: "EspressoHIP",
    products: [
        .library(name: "EspressoHIP", targets: ["EspressoHIP"]),
    ],
    targets: [
        // Sources/CEspressoHIP holds module.modulemap and espresso_hip.h (a copy or a symlink of include/espresso_hip.h).
        .systemLibrary(name: "CEspressoHIP", path: "Sources/CEspressoHIP"),
        .target(
            name: "EspressoHIP",
            dependencies: ["CEspressoHIP"],
            path: "Sources/EspressoHIP",
            linkerSettings: [
                // wherever espresso_amd/lib/libespresso_hip.so was installed
                .unsafeFlags(["-L/opt/espresso_amd/lib", "-Xlinker", "-rpath", "-Xlinker", "/opt/espresso_amd/lib"]),
                .linkedLibrary("espresso_hip"),
            ]
        ),
    ]
)
