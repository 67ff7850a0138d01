"""ntc_hip_decode_static (the decode entry point that allocates nothing: its mip table lives in an
array built into the library) against ntc_hip_decode, through the C ABI: every output byte equal, on
two calls in a row, the second with a smaller input, then a batch of sets; and the size limit."""
import numpy as np
import pytest

from cases import cfg_case, first_mismatch

pytestmark = pytest.mark.gpu

ACTIVE = (-17.0, -12.0)


def decode_both_ways(device, case):
    dset = case.device_set(device, fill=0xCD)
    device.decode([dset])
    device.synchronize()
    expected = case.d_output.download().copy()
    case.d_output.fill(0xCD)
    device.decode_static([dset])
    device.synchronize()
    got = case.d_output.download()
    return expected, got


def test_static_table_decode_equals_decode_twice_in_a_row(ntc, device):
    spec = ntc.presets.spec_cfg01()
    big = cfg_case(ntc, spec, 256, 256, 9, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=21, scale_log2_range=ACTIVE)
    small = cfg_case(ntc, spec, 100, 36, 3, 7, ntc.abi.OUT_UNORM8_PIXELS, seed=22, scale_log2_range=ACTIVE)
    for name, case in (("first call, 256x256 with 9 mips", big), ("second call, 100x36 with 3 mips", small)):
        expected, got = decode_both_ways(device, case)
        assert np.any(expected != 0xCD)
        mm = first_mismatch(expected, got)
        assert mm is None, f"{name}: {mm[1]} of {expected.size} bytes differ, first at {mm[0]}"


def test_static_table_decode_of_a_batch_spanning_several_table_chunks(ntc, device):
    """Five sets with eight mips each: 40 table entries, written by three table-writing launches."""
    spec = ntc.presets.spec_cfg2()
    cases = [cfg_case(ntc, spec, 128, 128, 8, 12, ntc.abi.OUT_UNORM8_PIXELS, seed=300 + i, scale_log2_range=ACTIVE)
             for i in range(5)]
    dsets = [c.device_set(device) for c in cases]
    device.decode(dsets)
    device.synchronize()
    expected = [c.d_output.download().copy() for c in cases]
    for c in cases:
        c.d_output.fill(0xCD)
    device.decode_static(dsets)
    device.synchronize()
    for i, c in enumerate(cases):
        assert first_mismatch(expected[i], c.d_output.download()) is None, f"set {i}"


def test_static_table_decode_rejects_more_mips_than_the_table_holds(ntc, device):
    spec = ntc.presets.spec_cfg01()
    case = cfg_case(ntc, spec, 64, 64, 7, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=5)
    dset = case.device_set(device)
    too_many = [dset] * 37                                   # 259 mips > 256
    with pytest.raises(ntc.NtcHipError) as err:
        device.decode_static(too_many)
    assert err.value.code == ntc.abi.ERR_INVALID_ARG and "built-in table" in err.value.message
    device.decode_static([dset] * 36)                        # 252 mips fit (the sets overlap; only the limit is tested)
    device.synchronize()


def test_static_table_decode_leaves_device_memory_as_it_is(ntc, device):
    """hipMemGetInfo before and after: ntc_hip_decode_static takes no device memory (and gives none back).  The first
    call of any kernel may make the runtime load code or set up its queue, so one call comes before the measurement."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    spec = ntc.presets.spec_cfg01()
    case = cfg_case(ntc, spec, 512, 512, 10, 16, ntc.abi.OUT_FP16_PLANAR_PAIRS, seed=23, scale_log2_range=ACTIVE)
    dset = case.device_set(device)
    device.decode_static([dset])
    device.synchronize()

    def free_bytes():
        free, total = C.c_size_t(0), C.c_size_t(0)
        assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    before = free_bytes()
    for _ in range(3):
        device.decode_static([dset])
    device.synchronize()
    assert free_bytes() == before
