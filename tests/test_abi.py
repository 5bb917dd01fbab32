"""The C-ABI library loads and exports exactly what ``include/dpk.h`` declares (no GPU needed)."""

import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "dpk.h"


def declared_functions():
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)  # strip comments
    names = re.findall(r"\b(dpk_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in [
        "dpk_linear_gs",
        "dpk_linear_bias_gs",
        "dpk_linear_ghost_norm",
        "dpk_conv2d_gs",
        "dpk_conv3d_gs",
        "dpk_embedding_bag_gs",
        "dpk_conv_bias_gs",
        "dpk_embedding_gs",
        "dpk_embedding_ghost_norm",
        "dpk_embedding_unique_pairs",
        "dpk_group_norm_gs",
        "dpk_rms_norm_gs",
        "dpk_layer_norm_gs",
        "dpk_sumsq_rows",
        "dpk_clip_factor",
        "dpk_clip_accumulate",
        "dpk_clip_accumulate_multi",
        "dpk_add_noise",
        "dpk_add_noise_multi",
        "dpk_clip_factor_per_layer",
        "dpk_clip_accumulate_per_layer",
    ]:
        assert must in names


def test_library_exports_every_declared_symbol():
    from opacus_amd import _lib

    assert _lib.LIB_PATH.exists(), "libdpsgd_hip.so is not built: run python -m opacus_amd.build"
    handle = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared_functions():
        assert hasattr(handle, name), f"{name} is declared in dpk.h but not exported"


def test_binding_covers_the_header_and_nothing_else():
    from opacus_amd import _lib

    assert sorted(_lib.SIGNATURES) == declared_functions()
    lib = _lib.lib()
    assert lib.dpk_abi_version() == _lib.ABI_VERSION


def test_binding_argument_counts_match_the_header():
    from opacus_amd import _lib

    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    for name, (_, argtypes) in _lib.SIGNATURES.items():
        m = re.search(r"\b" + name + r"\s*\((.*?)\)\s*;", text, flags=re.S)
        assert m, name
        args = m.group(1).strip()
        count = 0 if args in ("", "void") else len(args.split(","))
        assert count == len(argtypes), f"{name}: header has {count} arguments, binding {len(argtypes)}"


def test_workspace_queries_and_argument_errors_without_a_gpu():
    """Host-side checks run before any launch: they work (and fail loudly) with no device."""
    from opacus_amd import _lib

    lib = _lib.lib()
    assert lib.dpk_linear_gs_workspace_bytes(128, 1, 4096, 4096) == 0
    assert lib.dpk_linear_gs_workspace_bytes(16, 256, 1024, 1024) >= 16 * 8 * 8 * 4
    assert lib.dpk_sumsq_rows_workspace_bytes(4, 8192 * 3) >= 4 * 3 * 4
    assert lib.dpk_linear_ghost_norm_workspace_bytes(2, 512, 8, 8) >= 2 * 2 * 36 * 4
    assert lib.dpk_embedding_workspace_bytes(2, 100, 64) > 0
    # a bad shape is refused before anything touches a device
    rc = lib.dpk_linear_gs(None, None, 0, None, 0, None, 4, 0, 8, 8, 1.0, 0, None, 0, None)
    assert rc == -1 and b"dpk_linear_gs" in lib.dpk_last_error()
    rc = lib.dpk_add_noise(None, 0, None, 0, 16, 1.0, 1.0, 0, 0, 1, None)
    assert rc == -6
    rc = lib.dpk_clip_accumulate(None, 7, None, None, 0, 4, 16, 0, None)
    assert rc == -2
    with pytest.raises(_lib.DpkError, match="DPK_E_SHAPE"):
        _lib.check("dpk_conv2d_gs", lib.dpk_conv2d_gs(None, None, 0, None, 0, None, 1, 3, 4, 4, 4, 3, 3, 1, 1, 0, 0, 0, 0, 1, 1, 2, 1.0, None, 0, None))
    # a kernel choice outside the enum is refused
    assert lib.dpk_linear_gs(None, None, 0, None, 0, None, 4, 2, 8, 8, 1.0, 64, None, 0, None) == -6
    assert lib.dpk_linear_ghost_norm(None, None, 0, None, None, 4, 2, 8, 8, 1.0, 3, None, 0, None) == -6
    # the ghost-norm workspace covers either route whatever the caller later asks for
    thin = lib.dpk_linear_ghost_norm_workspace_bytes(4, 512, 16, 1024)
    assert thin >= lib.dpk_linear_gs_workspace_bytes(4, 512, 16, 1024) + 4 * 16 * 4
    # n == 0 is a no-op
    assert lib.dpk_linear_gs(None, None, 0, None, 0, None, 0, 1, 8, 8, 1.0, 0, None, 0, None) == 0
