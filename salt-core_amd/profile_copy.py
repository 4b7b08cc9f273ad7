"""A plain device-to-device copy of known size, run under `rocprofv3 --pmc` to
calibrate what the FETCH_SIZE / WRITE_SIZE counters read per byte moved."""
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))
from __graft_entry__ import load_package  # noqa: E402

if __name__ == "__main__":
    import ctypes as C
    gpu = load_package().lib
    lib = gpu.init()
    nbytes = 512 << 20
    src, dst = gpu.DeviceBuffer(nbytes, fill=1), gpu.DeviceBuffer(nbytes, fill=2)
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    for _ in range(3):
        assert hip.hipMemcpy(dst.ptr, src.ptr, nbytes, 3) == 0      # hipMemcpyDeviceToDevice
    print(f"copied {nbytes} bytes three times")
