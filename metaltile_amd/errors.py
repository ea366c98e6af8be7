"""Error type of the HIP backend.

Counterpart of ``MetalTileError`` (crates/metaltile-runtime/src/error.rs:8-55):
one exception carrying the C-ABI's negative code and its message.
"""

OK = 0
NO_DEVICE = -1
BAD_ARG = -2
SHAPE = -3
BUFFER_SIZE = -4
UNKNOWN_KERNEL = -5
HIP = -6
UNSUPPORTED = -7

_NAMES = {
    NO_DEVICE: "NoDevice", BAD_ARG: "Buffer", SHAPE: "Dispatch(shape)", BUFFER_SIZE: "BufferSize",
    UNKNOWN_KERNEL: "UnknownKernel", HIP: "Dispatch(hip)", UNSUPPORTED: "Unsupported",
}


class MtqError(RuntimeError):
    def __init__(self, code: int, message: str):
        self.code = code
        self.kind = _NAMES.get(code, "Unknown")
        super().__init__(f"{self.kind} ({code}): {message}")
