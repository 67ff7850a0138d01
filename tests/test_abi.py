"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol that
include/ntc_hip.h declares, its structs match the ctypes mirror, and compute entry points
fail loudly (never fall back) when no device was initialised."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ntc_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ntc_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(ntc):
    lib = ntc.load_library()
    names = declared_symbols()
    assert len(names) >= 15
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/ntc_hip.h but not exported"
    assert sorted(n for n, _, _ in ntc.abi.EXPORTS) == names


def test_struct_sizes_match_header(ntc, tmp_path):
    """Compiles a tiny C program against the header and compares sizeof/offsetof with ctypes."""
    src = tmp_path / "sizes.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "ntc_hip.h"\n'
        'int main(void){printf("%zu %zu %zu %zu %zu %zu %zu\\n", sizeof(NtcHipDecoderSpec), sizeof(NtcHipWeightLayout),'
        ' sizeof(NtcHipMipDesc), sizeof(NtcHipTextureSet), offsetof(NtcHipTextureSet, latents),'
        ' offsetof(NtcHipTextureSet, mips), offsetof(NtcHipMipDesc, hrOffset));return 0;}\n')
    exe = tmp_path / "sizes"
    import subprocess
    subprocess.run(["gcc", "-std=c99", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    got = [int(v) for v in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()]
    A = ntc.abi
    want = [C.sizeof(A.DecoderSpec), C.sizeof(A.WeightLayout), C.sizeof(A.MipDesc), C.sizeof(A.TextureSet),
            A.TextureSet.latents.offset, A.TextureSet.mips.offset, A.MipDesc.hrOffset.offset]
    assert got == want


def test_compute_entry_points_refuse_without_device(ntc):
    import importlib
    torch_spec = importlib.util.find_spec("torch")
    lib = ntc.load_library()
    rc = lib.ntc_hip_init(0)
    if rc == 0:
        pytest.skip("a HIP device is present; the no-device path is not reachable here")
    assert rc == ntc.abi.ERR_NO_DEVICE
    assert b"No HIP device" in lib.ntc_hip_last_error()
    sets = (ntc.abi.TextureSet * 1)()
    assert lib.ntc_hip_decode(sets, 1) == ntc.abi.ERR_NOT_INITIALIZED
    ms = C.c_float()
    assert lib.ntc_hip_decode_timed(sets, 1, 1, C.byref(ms)) == ntc.abi.ERR_NOT_INITIALIZED
    assert lib.ntc_hip_timer_begin() == ntc.abi.ERR_NOT_INITIALIZED
    assert lib.ntc_hip_timer_end(C.byref(ms)) == ntc.abi.ERR_NOT_INITIALIZED
    p = C.c_void_p()
    assert lib.ntc_hip_alloc(C.byref(p), 16) == ntc.abi.ERR_NOT_INITIALIZED
    with pytest.raises(ntc.NtcHipError):
        ntc.Device(0)
    assert torch_spec is None or True


def test_layout_helper_rejects_malformed_specs(ntc):
    lib = ntc.load_library()
    spec = ntc.presets.spec_cfg01()
    spec.hiddenChannels[1] = 40                      # not a multiple of 16
    out = ntc.abi.WeightLayout()
    assert lib.ntc_hip_weight_layout(spec, out) == ntc.abi.ERR_INVALID_ARG
    assert lib.ntc_hip_grid_bytes(256, 256, 8, 2) == 256 * 256 * 2
    assert lib.ntc_hip_grid_bytes(128, 128, 16, 4) == 128 * 128 * 8
    assert lib.ntc_hip_grid_bytes(128, 128, 12, 4) == 128 * 128 * 6
    assert lib.ntc_hip_grid_bytes(0, 128, 12, 4) == 0
