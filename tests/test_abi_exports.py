"""The C ABI library loads without a GPU and exports every function the header declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


HEADERS = ("eppgcn_hip.h", "eppgcn_hip_tuning.h")     # the drop-in surface; the process-wide tuning and test knobs


def declared_functions(headers=HEADERS):
    names = set()
    for header in headers:
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(eppgcn_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_tuning_knobs_stay_out_of_the_product_header():
    product = declared_functions(("eppgcn_hip.h",))
    assert not [n for n in product if n.startswith("eppgcn_set_") and n != "eppgcn_set_timing"]
    knobs = declared_functions(("eppgcn_hip_tuning.h",))
    assert knobs and all(n.startswith("eppgcn_set_") for n in knobs)


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
        assert hasattr(lib, name), f"{name} is declared under include/ but not exported"
    assert sorted(capi.EXPORTS) == declared_functions()
    assert capi.load().eppgcn_abi_version() == capi.ABI_VERSION


def test_host_only_heuristics_match_the_checker():
    """These two entry points are pure host code, so they can be compared without a GPU."""
    from eppgcn_amd import capi
    from oracle import c_oracle as co
    for vn, vl in [(1000, 5000), (100000, 1000000), (419000, 13400000), (3, 2000), (10, 5120)]:
        raw = co.map_back_part_size(vn, vl)
        assert capi.map_back_part_size(vn, vl) == (max(raw, 1), raw < 1)
        assert capi.threshold_back_part_size(vn, vl) == co.threshold_back_part_size(vn, vl)
    # the re-fitted rule: 16 below 24 kept edges per kept row, 32 from there on
    assert [capi.wave64_back_part_size(vn, vl) for vn, vl in [(0, 0), (10, 0), (10, 239), (10, 240), (3, 10 ** 9)]] == \
        [16, 16, 16, 32, 32]
    # the safe form of the `map` mode: the regression while it is usable, the wave64 rule where it is not
    assert capi.auto_back_part_size(1000, 5000) == (co.map_back_part_size(1000, 5000), False)
    assert co.map_back_part_size(10 ** 6, 10 ** 8) < 1 and capi.auto_back_part_size(10 ** 6, 10 ** 8) == (32, True)
    assert capi.auto_back_part_size(4 * 10 ** 6, 4 * 10 ** 7) == (16, True)
    assert capi.auto_back_part_size(0, 0) == (16, True)


def test_product_package_never_imports_the_checker():
    """The shipped package must not route through oracle/ (or any CPU fallback)."""
    pkg = os.path.join(ROOT, "eppgcn_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the checker"


def test_argument_errors_are_reported_before_any_device_work():
    """Invalid sizes and null pointers are rejected by host-side checks (return code -1 and a
    message naming the function), so these calls are safe without a GPU."""
    from eppgcn_amd import capi
    lib = capi.load()
    p0 = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)      # a non-null, aligned, never dereferenced address
    cases = [
        (lib.eppgcn_update_forward(one, 4, one, one, p0, 0, 8, 0, 5, p0), "in_dim > 0"),
        (lib.eppgcn_update_forward(one, 3, one, one, p0, 0, 8, 4, 5, p0), "ld_out"),
        (lib.eppgcn_update_forward(one, 8, one, p0, p0, 0, 8, 4, 5, p0), "null matrix"),
        (lib.eppgcn_update_backward_input(one, one, one, p0, -1, 4, 5, p0), "num_nodes >= 0"),
        (lib.eppgcn_update_backward_weight(one, one, one, 0, 8, 4, 5, p0, 0, p0), "workspace"),
        (lib.eppgcn_mark_compact(one, one, one, one, one, one, one, one, 3, 1 << 31, 0, one, 1 << 20, p0, None, p0),
         "num_edges"),
        (lib.eppgcn_mark_compact(one, one, one, one, one, one, one, one, 3, 100, 0, one, 8, p0, None, p0), "workspace too small"),
        (lib.eppgcn_spmm_forward(one, p0, p0, one, one, one, one, 8, 4, 2, 1, 1, 1, p0, 0, p0, p0), "null feature"),
        (lib.eppgcn_spmm_forward(one, one, p0, one, one, one, one, 8, 0, 2, 1, 1, 1, p0, 0, p0, p0), "dim > 0"),
    ]
    cases += [(lib.eppgcn_scan_status(ctypes.c_void_p(20), p0), "workspace"), (lib.eppgcn_plan_status(p0, 5, 9, 4, None, p0), "plan"),
              (lib.eppgcn_plan_status(one, -1, 0, 4, None, p0), "negative")]
    for rc, needle in cases:
        assert rc == -1
    # the message belongs to the last failing call
    assert b"negative" in lib.eppgcn_last_error()
    assert lib.eppgcn_plan_status(p0, 0, 0, 4, None, p0) == 0
    lib.eppgcn_plan_release(p0)           # both are no-ops for a plan the library does not know
    lib.eppgcn_plan_release(one)
    # a plan the library has not seen is sized like the plain feature workspace
    assert lib.eppgcn_plan_workspace_floats(one, 10, 22) == lib.eppgcn_feature_workspace_floats(10, 22) == 4096 * 32
    assert [lib.eppgcn_feature_workspace_row(r) for r in (0, 31, 32, 4095, 4096, 131072 + 64)] == [0, 31, 33, 4095 ^ 127, 4096 ^ 128, (131072 + 64) ^ 2]
    assert lib.eppgcn_update_supported(96, 16) == 7 and lib.eppgcn_update_supported(2000, 16) == 6
    assert lib.eppgcn_update_supported(16, 100) == 3 and lib.eppgcn_update_supported(0, 4) == 0
    assert lib.eppgcn_feature_workspace_pitch(16) == 16 and lib.eppgcn_feature_workspace_pitch(22) == 32
    assert lib.eppgcn_feature_workspace_pitch(3) == 4 and lib.eppgcn_feature_workspace_pitch(40) == 40
    assert lib.eppgcn_update_workspace_bytes(0, 4, 4) == 0
    assert lib.eppgcn_mark_compact_workspace_bytes(4096 * 3 + 1) >= 32 + 8 * 4 + 4 * 5


def test_header_is_plain_c_and_a_c_program_links_against_the_library(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 and as C++ without torch or HIP
    headers, and a C program must link against the library and call it.  Only host-side entry
    points are called here (no GPU)."""
    import subprocess
    from eppgcn_amd import capi
    inc = os.path.join(ROOT, "include")
    src = tmp_path / "client.c"
    src.write_text(
        '#include "eppgcn_hip.h"\n'
        "#include <stdio.h>\n"
        "int main(void) {\n"
        "    int clamped = 0;\n"
        "    int ps = eppgcn_map_back_part_size(1000, 5000, &clamped);\n"
        '    printf("%d %d %zu %d %d %d\\n", eppgcn_abi_version(), eppgcn_feature_workspace_pitch(22),\n'
        "           eppgcn_feature_workspace_floats(10, 22), ps, clamped,\n"
        "           eppgcn_spmm_forward(0, 0, 0, 0, 0, 0, 0, 4, 0, 0, 1, 1, 1, 0, 0, 0, 0));\n"
        '    printf("%s\\n", eppgcn_last_error());\n'
        "    return 0;\n"
        "}\n")
    for compiler, std in (("gcc", "-std=c99"), ("g++", "-std=c++11")):
        subprocess.run([compiler, std, "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", "-x",
                        "c" if compiler == "gcc" else "c++", "-I", inc, str(src)], check=True)
    exe = tmp_path / "client"
    libdir = os.path.dirname(capi.LIB_PATH)
    subprocess.run(["gcc", "-std=c99", "-I", inc, str(src), "-o", str(exe), "-L", libdir, "-leppgcn_hip",
                    "-Wl,-rpath," + libdir, "-Wl,-rpath-link,/opt/rocm/lib"], check=True)
    env = dict(os.environ, LD_LIBRARY_PATH="/opt/rocm/lib:" + os.environ.get("LD_LIBRARY_PATH", ""))
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True, env=env).stdout.split("\n")
    from oracle import c_oracle as co
    assert out[0].split() == [str(capi.ABI_VERSION), "32", str(4096 * 32), str(max(1, co.map_back_part_size(1000, 5000))), "0", "-1"]
    assert "dim > 0" in out[1]
