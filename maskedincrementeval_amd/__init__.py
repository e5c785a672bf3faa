"""MI355X-native masked incremental inference (drop-in for the reference's incr_modules).

    masked_types            Masked / DenseT aliases, TileMask
    mask_incr_functional    IncrementReserve + functional ops
    mask_incr_modules       nn.Module surface (nnConvIncr, nnReservedActivation, ...)
    e2depth_incr            E2Depth-incr network built from the modules
    ops / _lib              tensor-level wrappers / ctypes binding of libmie_hip.so

All compute runs in hand-written HIP kernels (csrc/) behind the C ABI of
include/mie.h; there is no eager or CPU fallback.
"""
__version__ = "0.1.0"
