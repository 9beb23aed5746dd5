// swift-tools-version: 5.9
// SwiftPM manifest of the target a swift-lm maintainer adds next to MetalCompiler.
// Not compiled in this repository's build: the build image has no Swift toolchain.  It binds
// the C ABI of include/mi355_qlinear.h (libmi355_qlinear.so) and exposes the value types the
// quantized-linear step of MetalCompiler consumes.
import PackageDescription

let package = Package(
    name: "MI355QuantizedLinear",
    products: [
        .library(name: "MI355QuantizedLinear", targets: ["MI355QuantizedLinear"]),
    ],
    targets: [
        // System-library style C target: module map over the installed header, links the .so.
        .target(
            name: "CMI355QLinear",
            path: "Sources/CMI355QLinear",
            publicHeadersPath: "include",
            linkerSettings: [.linkedLibrary("mi355_qlinear")]
        ),
        .target(
            name: "MI355QuantizedLinear",
            dependencies: ["CMI355QLinear"],
            path: "Sources/MI355QuantizedLinear"
        ),
    ]
)
