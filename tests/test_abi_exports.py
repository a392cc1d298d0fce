"""The C ABI library loads without a GPU and exports every function the header declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "eppgcn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(eppgcn_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ("eppgcn_spmm_forward", "eppgcn_spmm_backward", "eppgcn_ours_backward", "eppgcn_mask_forward",
                 "eppgcn_compact_back_edge", "eppgcn_split_back_part", "eppgcn_build_part",
                 "eppgcn_count_nonzero", "eppgcn_map_back_part_size", "eppgcn_get_ginfo",
                 "eppgcn_print_time", "eppgcn_clear_time"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from eppgcn_amd import capi
    assert os.path.exists(capi.LIB_PATH), "build the library first: python -m eppgcn_amd.build"
    lib = ctypes.CDLL(capi.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/eppgcn_hip.h but not exported"
    assert sorted(capi.EXPORTS) == declared_functions()
    assert capi.load().eppgcn_abi_version() == 4


def test_host_only_heuristics_match_the_checker():
    """These two entry points are pure host code, so they can be compared without a GPU."""
    from eppgcn_amd import capi
    from oracle import c_oracle as co
    for vn, vl in [(1000, 5000), (100000, 1000000), (419000, 13400000), (3, 2000), (10, 5120)]:
        raw = co.map_back_part_size(vn, vl)
        assert capi.map_back_part_size(vn, vl) == (max(raw, 1), raw < 1)
        assert capi.threshold_back_part_size(vn, vl) == co.threshold_back_part_size(vn, vl)


def test_product_package_never_imports_the_checker():
    """The shipped package must not route through oracle/ (or any CPU fallback)."""
    pkg = os.path.join(ROOT, "eppgcn_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the checker"
