"""Contexts of the C ABI (ntc_hip_create / ntc_hip_destroy / ntc_hip_ctx_*): each owns its stream, its mip
table and its loss partials, so two of them on one device decode different sets interleaved without
disturbing each other, byte-equal to the checker; the default context keeps working beside them."""
import ctypes as C

import numpy as np
import pytest

from cases import cfg_case, ref_case, first_mismatch

ACTIVE = (-17.0, -12.0)


def test_context_entry_points_refuse_null_and_destroyed_contexts(ntc):
    lib = ntc.load_library()
    sets = (ntc.abi.TextureSet * 1)()
    assert lib.ntc_hip_ctx_decode(None, sets, 1) == ntc.abi.ERR_NOT_INITIALIZED
    assert b"context is null" in lib.ntc_hip_last_error()
    assert lib.ntc_hip_ctx_synchronize(None) == ntc.abi.ERR_NOT_INITIALIZED
    p = C.c_void_p()
    assert lib.ntc_hip_ctx_alloc(None, C.byref(p), 16) == ntc.abi.ERR_NOT_INITIALIZED
    lib.ntc_hip_destroy(None)                                    # allowed
    assert lib.ntc_hip_create(0, None) == ntc.abi.ERR_INVALID_ARG


@pytest.mark.gpu
def test_two_contexts_decode_different_sets_interleaved(ntc, device):
    a, b = ntc.Device(0, own_context=True), ntc.Device(0, own_context=True)
    try:
        spec_a, spec_b = ntc.presets.spec_cfg01(), ntc.presets.spec_ref092(12)
        case_a = cfg_case(ntc, spec_a, 256, 128, 8, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=71, scale_log2_range=ACTIVE)
        case_b = ref_case(ntc, spec_b, 192, 192, 8, 3, 10, ntc.abi.OUT_UNORM8_PIXELS, seed=72, scale_log2_range=ACTIVE)
        case_d = cfg_case(ntc, ntc.presets.spec_cfg2(), 128, 128, 8, 12, ntc.abi.OUT_FP16_PIXELS, seed=73, scale_log2_range=ACTIVE)
        hosts = [c.host_set() for c in (case_a, case_b, case_d)]
        for h in hosts:
            h.decode(threads=8)
        set_a, set_b, set_d = case_a.device_set(a), case_b.device_set(b), case_d.device_set(device)
        for _ in range(4):                                        # no synchronisation in between: three streams, three mip tables
            a.decode([set_a])
            b.decode([set_b])
            device.decode([set_d])
        # a loss pass on each context as well (partial sums are per context)
        mse_a, mse_b = (C.c_float * 16)(), (C.c_float * 16)()
        mip = case_a.mips[0]
        planar_bytes = mip.width * mip.height * 16 * 2
        a.call("image_loss", case_a.d_output.ptr, case_a.d_output.ptr, planar_bytes, mip.width, mip.height, 16, 0xFFFF, -1, 0, mse_a)
        other = b.upload(np.zeros(planar_bytes // 2, dtype=np.uint16))
        b.call("image_loss", other.ptr, other.ptr, planar_bytes, mip.width, mip.height, 16, 0xFFFF, -1, 0, mse_b)
        assert list(mse_a) == [0.0] * 16 and list(mse_b) == [0.0] * 16
        a.synchronize(); b.synchronize(); device.synchronize()
        for case, host, name in ((case_a, hosts[0], "context a"), (case_b, hosts[1], "context b"), (case_d, hosts[2], "default context")):
            mm = first_mismatch(host.output, case.d_output.download())
            assert mm is None, f"{name}: {mm[1]} bytes differ, first at {mm[0]}"
        # a destroyed context is refused, the others go on
        for buf in (case_a.d_latents, case_a.d_weights, case_a.d_output):
            buf.free()
        a.close()
        b.decode([set_b])
        b.synchronize()
        assert first_mismatch(hosts[1].output, case_b.d_output.download()) is None
        other.free()
    finally:
        for case in (case_b,):
            for buf in (case.d_latents, case.d_weights, case.d_output):
                buf.free()
        a.close()
        b.close()
