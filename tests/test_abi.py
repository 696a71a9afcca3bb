"""The C-ABI library loads without a GPU, exports every symbol the header
declares, and rejects invalid arguments before touching the device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mccnn_hip.h")
LIB = os.path.join(ROOT, "tensorflow_graphics_point_clouds_amd", "libmccnn_hip.so")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        pytest.fail("libmccnn_hip.so is not built; run __graft_entry__.build()")
    handle = ctypes.CDLL(LIB)
    handle.mccnn_last_error.restype = ctypes.c_char_p
    return handle


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mccnn_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    names = declared_symbols()
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_abi_version(lib):
    assert lib.mccnn_abi_version() == 1


def test_invalid_arguments_return_status_not_abort(lib):
    i64 = ctypes.c_int64
    rc = lib.mccnn_compute_keys(None, i64(10), 7, None, i64(10), None, i64(1), 7, None, 7, None,
                                7, None, None)
    assert rc == 1 and b"dimension" in lib.mccnn_last_error()
    rc = lib.mccnn_compute_keys(None, i64(10), 3, None, i64(9), None, i64(1), 3, None, 3, None,
                                3, None, None)
    assert rc == 1 and b"batch ids" in lib.mccnn_last_error()
    # K must be 8/16/32/64, C < 8 or a multiple of 8, pairs need two columns
    args = lambda k, c, cols: (None, i64(5), k, None, i64(4), c, None, i64(5), 2, cols, None,
                               i64(3), None, None)
    assert lib.mccnn_basis_proj(*args(12, 8, 2)) == 1
    assert lib.mccnn_basis_proj(*args(8, 12, 2)) == 1
    assert lib.mccnn_basis_proj(*args(8, 8, 3)) == 1
    # sampling and pdf modes
    total = i64(0)
    rc = lib.mccnn_sampling_count(None, 2, i64(4), 3, None, i64(4), None, i64(4), None, 3, None,
                                  i64(4), 2, 2, None, i64(4), None, None, ctypes.c_size_t(0),
                                  ctypes.byref(total))
    assert rc == 1 and b"mode" in lib.mccnn_last_error()
    rc = lib.mccnn_compute_pdf(None, i64(4), 3, None, i64(4), 2, 2, None, i64(5), None, 3, None,
                               3, None, 0, None)
    assert rc == 1 and b"same points as samples" in lib.mccnn_last_error()
    host = (ctypes.c_int32 * 3)(1, 1, 1)
    rc = lib.mccnn_build_grid_ds(None, i64(4), None, 3, None, 3, host, 0, None)
    assert rc == 1 and b"batch size" in lib.mccnn_last_error()


def test_pointconv_density_entry_points_validate_before_the_device(lib):
    i64, sz = ctypes.c_int64, ctypes.c_size_t
    rc = lib.mccnn_pointconv_density(None, i64(5), None, 2, None, None, None, None, None, None, None)
    assert rc == 1 and b"point_column" in lib.mccnn_last_error()
    assert lib.mccnn_pointconv_density(None, i64(0), None, 0, None, None, None, None, None, None,
                                       None) == 0
    rc = lib.mccnn_pointconv_density_grads(None, i64(5), None, 0, None, None, None, None, None, None,
                                           None, 5, None, None, sz(0), None)
    assert rc == 1 and b"slabs" in lib.mccnn_last_error()
    lib.mccnn_pointconv_density_grads_workspace_bytes.restype = sz
    assert lib.mccnn_pointconv_density_grads_workspace_bytes(i64(10 ** 6)) >= 49 * 4


def test_layer_entry_points_reject_uncovered_shapes(lib):
    i64, sz = ctypes.c_int64, ctypes.c_size_t
    assert lib.mccnn_mc_conv_supported(3, 64, 16) == 1 and lib.mccnn_mc_conv_supported(3, 24, 16) == 0
    assert lib.mccnn_mc_conv_layer_supported(3, 64, 16, 64) == 1
    assert lib.mccnn_mc_conv_layer_supported(4, 64, 16, 64) == 0
    assert lib.mccnn_weight_grad_product_supported(64, 1024) == 1
    assert lib.mccnn_weight_grad_product_supported(48, 1024) == 0
    assert lib.mccnn_projection_grad_product_supported(64, 1024) == 1
    assert lib.mccnn_projection_grad_product_supported(128, 1024) == 1
    assert lib.mccnn_projection_grad_product_supported(96, 1024) == 0
    assert lib.mccnn_final_product_supported(2048, 128) == 1
    assert lib.mccnn_final_product_supported(1000, 128) == 0
    # K = 8 is not covered by the fused projection
    rc = lib.mccnn_mc_conv_project(None, 3, i64(10), None, 64, None, i64(10), None, i64(20), None,
                                   None, None, 8, 1, 0, None, None, None, None, None)
    assert rc == 1 and b"K in {16,32,64}" in lib.mccnn_last_error()
    assert lib.mccnn_mc_conv_project_supported(3, 48, 32) == 1
    assert lib.mccnn_mc_conv_weight_grads_supported(3, 64, 64) == 1
    assert lib.mccnn_mc_conv_supported(3, 64, 32) == 0          # no feature-gradient half there
    rc = lib.mccnn_kp_conv_project(None, 3, i64(10), None, 64, None, i64(10), None, i64(20), None,
                                   None, None, 33, None, 0, ctypes.c_float(1.0), None, None)
    assert rc == 1 and b"kernel points" in lib.mccnn_last_error()
    rc = lib.mccnn_weight_grad_product(None, i64(10), 48, None, 1024, None, None, sz(0), None)
    assert rc == 1 and b"output rows" in lib.mccnn_last_error()
    rc = lib.mccnn_projection_grad_product(None, i64(10), 96, None, 1024, None, None)
    assert rc == 1 and b"input columns" in lib.mccnn_last_error()
    # a feature table too large for 32-bit byte offsets is refused, not truncated
    rc = lib.mccnn_mc_conv_project(None, 3, i64(1 << 25), None, 64, None, i64(10), None, i64(20),
                                   None, None, None, 16, 1, 0, None, None, None, None, None)
    assert rc == 1 and b"2^30" in lib.mccnn_last_error()
    fn = lib.mccnn_mc_conv_project_grads_workspace_bytes
    fn.restype = sz
    assert fn(3, 16, i64(1000)) >= 32 * 64 * 4


def test_workspace_queries(lib):
    for name in ("mccnn_sort_keys_workspace_bytes", "mccnn_sampling_workspace_bytes"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_size_t
        assert fn(ctypes.c_int64(1000)) > 1000 * 4
    fn = lib.mccnn_find_neighbors_workspace_bytes
    fn.restype = ctypes.c_size_t
    assert fn(3, ctypes.c_int64(1000)) >= 1000 * 9 * 8
    assert fn(9, ctypes.c_int64(1000)) == 0


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "tensorflow_graphics_point_clouds_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(base, f)).read()
                assert "mccnn_oracle" not in text and "from oracle" not in text, f
