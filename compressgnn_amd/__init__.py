"""MI355X-native implementation of the CompressGNN runtime hot path.

Sub-modules:
  abi      ctypes view of the device library's C ABI (libcgnn_hip.so)
  build    build recipes for the native parts
  layer/   drop-in layer modules (same file and class names as the reference's layer/)
  loader/  drop-in loader modules (CompressGraph, CompressgnnData)
"""
__version__ = "0.1.0"
