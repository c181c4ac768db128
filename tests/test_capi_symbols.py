"""CPU-side checks of the drop-in boundary: the library loads and exports exactly
the entry points include/lbnorm.h declares, and the Python binding lists the same."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "lbnorm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lbn_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for layer in ("layer_norm", "batch_norm", "softmax", "log_softmax", "channelwise_softmax"):
        assert f"lbn_{layer}_fwd_f32" in names and f"lbn_{layer}_bwd_f32" in names
    assert "lbn_layer_norm_fwd_f16" in names and "lbn_layer_norm_bwd_f16" in names
    # the five layers also exist for TensorDataType = double
    for layer in ("layer_norm", "batch_norm", "softmax", "log_softmax", "channelwise_softmax"):
        assert f"lbn_{layer}_fwd_f64" in names and f"lbn_{layer}_bwd_f64" in names


def test_library_exports_every_declared_symbol():
    from lbann_amd import capi
    assert os.path.exists(capi.LIB_PATH), "run `python -m lbann_amd.build` first"
    handle = ctypes.CDLL(capi.LIB_PATH)
    for name in declared_functions():
        assert hasattr(handle, name), f"{name} is declared in lbnorm.h but not exported"


def test_binding_matches_header():
    from lbann_amd import capi
    assert sorted(capi.PROTOTYPES) == declared_functions()
    lib = capi.lib()
    assert lib.lbn_version() >= 100
    assert lib.lbn_status_string(0) == b"ok"
    # size queries are pure host arithmetic and need no device
    assert lib.lbn_softmax_workspace_bytes(262144, 16) >= 16 * 8
    assert lib.lbn_softmax_workspace_bytes(0, 16) == 0
    assert lib.lbn_batch_norm_workspace_bytes(256, 3136, 64) > 0
    assert lib.lbn_layer_norm_bwd_workspace_bytes(1, 4096, 8192, 0, 2) == 0
    assert lib.lbn_layer_norm_fwd_workspace_bytes(1, 4096, 8192, 2) == 0
    assert lib.lbn_layer_norm_fwd_workspace_bytes(1, 802816, 64, 4) >= 64 * 49 * 16     # slots of 64 rows x 49 workgroups
    assert lib.lbn_layer_norm_bwd_workspace_bytes(1, 802816, 64, 0, 4) >= 64 * 98 * 16
    assert lib.lbn_layer_norm_bwd_workspace_bytes(1, 802816, 64, 1, 4) >= 2 * 2 * 802816 * 4
    assert lib.lbn_layer_norm_bwd_workspace_bytes(1, 4096, 8192, 1, 2) >= 2 * 4096 * 4


def test_host_mirror_dimension_logic():
    """get_normdims / get_channel_size_and_stride restated on the host (no device needed)."""
    from lbann_amd import layers as L
    cw = L.channelwise_softmax_layer.__new__(L.channelwise_softmax_layer)
    cw.dims, cw.m_dim, cw.m_single_dim_mode = (5, 2, 7), 0, False
    assert cw.get_channel_size_and_stride() == (14, 14, 5)
    cw.m_dim, cw.m_single_dim_mode = -1, True
    assert cw.get_channel_size_and_stride() == (7, 7, 10)
    cw.dims, cw.m_dim, cw.m_single_dim_mode = (64, 4096), 0, False
    assert cw.get_channel_size_and_stride() == (4096, 4096, 64)


def test_header_is_plain_c(tmp_path):
    """include/lbnorm.h compiles as C99 and as C++17 on its own (no HIP, no torch types)."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "use_header.c"
    src.write_text('#include "lbnorm.h"\nint (*entry)(void) = lbn_version;\nint main(void) { return entry ? LBN_OK : LBN_ERR_UNSUPPORTED; }\n')
    inc = os.path.join(root, "include")
    subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only", f"-I{inc}", str(src)], check=True)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", f"-I{inc}", str(src)], check=True)
