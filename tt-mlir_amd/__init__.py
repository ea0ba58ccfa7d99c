"""MI355X-native execution backend for tt-mlir TTNN programs (host-side Python mirror).

The package directory name contains a hyphen, so it is loaded by path under the module name
`ttmlir_amd` (see __graft_entry__.load_package).  Sub-modules:

  hip       ctypes binding of lib/libttmlir_amd_hip.so (the C ABI over the gfx950 kernels)
  datagen   seeded synthetic inputs of the benchmark configurations
  build     in-tree build of the native libraries
"""
__all__ = ["hip", "datagen", "build"]
