"""The C-ABI library loads and exports every symbol that include/tosa_mi355.h declares (no GPU needed)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tosa_mi355.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tmi_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_path():
    names = declared_functions()
    for want in ("tmi_conv2d", "tmi_depthwise_conv2d", "tmi_matmul", "tmi_rescale", "tmi_clamp",
                 "tmi_conv2d_rescale_clamp", "tmi_depthwise_conv2d_rescale_clamp", "tmi_ctx_create",
                 "tmi_ctx_sync", "tmi_buf_alloc", "tmi_upload", "tmi_download"):
        assert want in names


def test_library_exports_every_declared_symbol():
    from reference_model_amd import capi
    lib = capi.load_library()
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, f"declared in the header but not exported: {missing}"
    assert sorted(capi.EXPORTS) == declared_functions()
    assert b"gfx950" in lib.tmi_version()


def test_structs_match_header_sizes():
    from reference_model_amd import capi
    # the int32 fields of each descriptor in include/tosa_mi355.h
    assert ctypes.sizeof(capi.ConvDesc) == 4 * 21
    assert ctypes.sizeof(capi.TconvDesc) == 4 * 19
    assert ctypes.sizeof(capi.Conv3dDesc) == 4 * 28
    assert ctypes.sizeof(capi.PoolDesc) == 4 * 17
    assert ctypes.sizeof(capi.RescaleDesc) == 4 * 11
    assert ctypes.sizeof(capi.Level) == 4 * 5


def test_no_cpu_fallback_without_device():
    """Without a GPU the context refuses to come up instead of computing anything on the host."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from reference_model_amd import Context
    with pytest.raises(RuntimeError):
        Context(0)


def test_build_refuses_kernels_with_a_scratch_segment():
    """the build reads the compiler's resource remarks and stops at a kernel that spills or indexes a register array at
    run time (such kernels were measured 1.5 to 2.5 times slower on the GPU)"""
    from reference_model_amd.build import kernels_with_scratch
    remarks = "\n".join([
        "a.hip:9:1: remark: Function Name: _Z4goodPi [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:9:1: remark:     VGPRs: 12 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:9:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:20:1: remark: Function Name: _Z5spillPi [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:20:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:20:1: remark:     ScratchSize [bytes/lane]: 184 [-Rpass-analysis=kernel-resource-usage]",
    ])
    assert kernels_with_scratch(remarks) == ["_Z5spillPi: 184 bytes per lane"]
    assert kernels_with_scratch("") == []
