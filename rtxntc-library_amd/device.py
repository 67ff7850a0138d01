"""Device-side plumbing over the C ABI: buffers, texture-set assembly, decode calls."""
import ctypes as C

import numpy as np

from . import abi, presets


class Device:
    """The library's default context (ntc_hip_init) or, with own_context=True, a context of its own
    (ntc_hip_create: its own stream and working memory); raises NtcHipError when there is no gfx950 device."""

    def __init__(self, index=0, own_context=False):
        self.lib = abi.load_library()
        self.ctx = None
        if own_context:
            handle = C.c_void_p()
            abi.check(self.lib.ntc_hip_create(index, C.byref(handle)))
            self.ctx = handle
        else:
            abi.check(self.lib.ntc_hip_init(index))
        name = C.create_string_buffer(256)
        cus = C.c_int(0)
        self.call("device_info", name, 256, C.byref(cus))
        self.name = name.value.decode()
        self.compute_units = cus.value
        khz = C.c_int(0)
        self.call("device_clock", C.byref(khz))
        self.clock_ghz = khz.value / 1e6

    def call(self, name, *args):
        """ntc_hip_<name>(args) on the default context, ntc_hip_ctx_<name>(context, args) on an own one."""
        if self.ctx is None:
            abi.check(getattr(self.lib, "ntc_hip_" + name)(*args))
        else:
            abi.check(getattr(self.lib, "ntc_hip_ctx_" + name)(self.ctx, *args))

    def close(self):
        if self.ctx is not None:
            self.lib.ntc_hip_destroy(self.ctx)
            self.ctx = None

    def alloc(self, nbytes):
        return DeviceBuffer(self, nbytes)

    def upload(self, array):
        array = np.ascontiguousarray(array)
        buf = DeviceBuffer(self, array.nbytes)
        self.call("upload", buf.ptr, array.ctypes.data, array.nbytes)
        return buf

    def synchronize(self):
        self.call("synchronize")

    @staticmethod
    def pack_sets(sets):
        """A C array of texture sets, reusable across decode calls."""
        return sets if isinstance(sets, C.Array) else (abi.TextureSet * len(sets))(*sets)

    def decode(self, sets):
        arr = self.pack_sets(sets)
        self.call("decode", arr, len(arr))

    def decode_static(self, sets):
        """ntc_hip_decode_static: the same decode with the mip table in the library's built-in array."""
        arr = self.pack_sets(sets)
        self.call("decode_static", arr, len(arr))

    def decode_timed(self, sets, iterations):
        arr = self.pack_sets(sets)
        ms = C.c_float(0)
        self.call("decode_timed", arr, len(arr), iterations, C.byref(ms))
        return ms.value


    def timer_begin(self):
        """ntc_hip_timer_begin: a HIP event on the context's stream in front of what is queued next."""
        self.call("timer_begin")

    def timer_end(self):
        """ntc_hip_timer_end: milliseconds of device time since timer_begin (waits for the queued work)."""
        ms = C.c_float(0)
        self.call("timer_end", C.byref(ms))
        return ms.value


class DeviceBuffer:
    def __init__(self, device, nbytes):
        self.device = device
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        device.call("alloc", C.byref(p), self.nbytes)
        self.ptr = p.value

    def download(self, dtype=np.uint8):
        out = np.empty(self.nbytes, dtype=np.uint8)
        self.device.call("download", out.ctypes.data, self.ptr, self.nbytes)
        return out.view(dtype)

    def download_range(self, offset, nbytes, dtype=np.uint8):
        assert 0 <= offset and offset + nbytes <= self.nbytes
        out = np.empty(int(nbytes), dtype=np.uint8)
        self.device.call("download", out.ctypes.data, self.ptr + int(offset), int(nbytes))
        return out.view(dtype)

    def fill(self, value):
        self.device.call("memset", self.ptr, value, self.nbytes)

    def free(self):
        if self.ptr:
            self.device.call("free", self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def make_texture_set(spec, mips, num_channels, output_format, latents_ptr, latents_bytes,
                     weights_ptr, weights_bytes, output_ptr, output_bytes, pixel_stride=0):
    """Fills an abi.TextureSet from already-placed buffers (device or host addresses)."""
    ts = abi.TextureSet()
    ts.spec = spec.copy()
    ts.numMips = len(mips)
    ts.numChannels = num_channels
    ts.outputFormat = output_format
    ts.outPixelStride = pixel_stride
    ts.latents, ts.weights, ts.output = latents_ptr, weights_ptr, output_ptr
    ts.latentsBytes, ts.weightsBytes, ts.outputBytes = latents_bytes, weights_bytes, output_bytes
    for i, d in enumerate(mips):
        C.memmove(C.byref(ts.mips[i]), C.byref(d), C.sizeof(abi.MipDesc))
    return ts
