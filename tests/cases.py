"""Builds matched host (oracle) and device (HIP) texture sets from one seeded description."""
import numpy as np


class Case:
    def __init__(self, ntc, spec, mips, latent_bytes, num_channels, output_format, seed,
                 scale_log2_range=(-10.0, -4.0), pixel_stride=None, weights=None, latents=None):
        self.ntc = ntc
        self.spec = spec
        self.mips = mips
        self.num_channels = num_channels
        self.output_format = output_format
        self.pixel_stride, self.output_bytes = ntc.presets.assign_output_offsets(mips, num_channels, output_format, pixel_stride)
        self.latents = latents if latents is not None else ntc.synth.make_latents(latent_bytes, seed)
        self.weights = weights if weights is not None else ntc.synth.make_weights(spec, seed + 1, scale_log2_range)
        self.texels = sum(d.width * d.height for d in mips)

    def host_set(self):
        from oracle_lib import HostSet
        return HostSet(self.ntc, self.spec, self.mips, self.num_channels, self.output_format,
                       self.latents, self.weights, self.output_bytes, self.pixel_stride)

    def device_set(self, device, fill=0xCD):
        self.d_latents = device.upload(self.latents)
        self.d_weights = device.upload(self.weights)
        self.d_output = device.alloc(self.output_bytes)
        self.d_output.fill(fill)
        return self.ntc.make_texture_set(
            self.spec, self.mips, self.num_channels, self.output_format,
            self.d_latents.ptr, self.d_latents.nbytes, self.d_weights.ptr, self.d_weights.nbytes,
            self.d_output.ptr, self.d_output.nbytes, self.pixel_stride)


def cfg_case(ntc, spec, width, height, num_mips, num_channels, output_format, seed, **kw):
    mips, latent_bytes = ntc.presets.mips_private_grids(spec, width, height, num_mips)
    return Case(ntc, spec, mips, latent_bytes, num_channels, output_format, seed, **kw)


def ref_case(ntc, spec, width, height, num_mips, grid_scale, num_channels, output_format, seed, **kw):
    mips, latent_bytes = ntc.presets.mips_ref092(spec, width, height, num_mips, grid_scale)
    return Case(ntc, spec, mips, latent_bytes, num_channels, output_format, seed, **kw)


def first_mismatch(a, b):
    a = np.asarray(a).reshape(-1)
    b = np.asarray(b).reshape(-1)
    bad = np.nonzero(a != b)[0]
    return None if bad.size == 0 else (int(bad[0]), int(bad.size), a[bad[0]], b[bad[0]])
