"""MI355X (gfx950) implementation of libnd4j's legacy op-execution path behind the NativeOps boundary.

``native``     ctypes binding of libnd4j_amd.so (the C ABI of include/nd4j_native_c.h); loading fails loudly
               when the library has not been built - there is no CPU fallback.
``harness``    what a host of the library does around a call: device buffers, shapeInfo, TAD tables and the
               extraPointers array.
``workloads``  the benchmark configurations.
"""
