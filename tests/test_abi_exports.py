"""The C-ABI library loads without a GPU and exports every symbol that include/grab_anns.h declares."""
import ctypes as C
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "grab_anns.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(grab_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(grab):
    names = _declared()
    assert len(names) > 50
    missing = [n for n in names if not hasattr(grab.lib, n)]
    assert not missing, f"declared in grab_anns.h but not exported: {missing}"


def test_host_only_calls_work_without_gpu(grab):
    assert grab.lib.grab_next_power_of_2(300) == 512
    assert grab.lib.grab_queue_capacity(64, 4, 64) == 512
    assert grab.lib.grab_reference_smem_bytes(64, 128, 4, 64, 13) == 37648
    assert 0 < grab.lib.grab_search_lds_bytes(64, 128, 4, 64, 64, 13) <= 160 * 1024
    assert grab.search_plan(grab.WRAP_SEARCH, 10, 32, 4, 64) == (64, 8, 512)
    assert grab.device_count() >= 0
    assert isinstance(grab.lib.grab_last_error(), bytes)


def test_argument_errors_do_not_need_a_gpu(grab):
    # validation happens on the host before anything is launched
    d = grab.SearchDesc()
    assert grab.lib.grab_search_ex(C.byref(d)) == 1
    assert b"Graph is null" in grab.lib.grab_last_error()
    assert grab.lib.grab_search_ex(None) == 1
    assert grab.lib.grab_sort_pairs(None, None, C.c_size_t(4)) == 1
    assert grab.lib.grab_vmm_resize(None, C.c_size_t(1)) == 1
    # the exact scans: null arrays, k beyond 128, a dimension that is no multiple of 4, an index that does not exist
    null = C.c_void_p(None)
    assert grab.lib.grab_window_scan_topk(null, C.c_size_t(10), C.c_uint32(8), null, C.c_size_t(1), C.c_uint32(1), C.c_int(0), null, null,
                                          null, null, None, None) == 1
    assert b"null pointer" in grab.lib.grab_last_error()
    fake = C.c_void_p(16)   # never dereferenced: the checks below fail first
    assert grab.lib.grab_window_scan_topk(fake, C.c_size_t(10), C.c_uint32(8), fake, C.c_size_t(1), C.c_uint32(129), C.c_int(0), fake, fake,
                                          fake, fake, None, None) == 1
    assert b"k must be in [1,128]" in grab.lib.grab_last_error()
    assert grab.lib.grab_bucket_scan_topk(fake, C.c_size_t(10), C.c_uint32(6), fake, C.c_uint32(1), fake, C.c_size_t(1), C.c_uint32(1),
                                          C.c_int(0), fake, fake, fake, None, None) == 1
    assert grab.lib.grab_scan_base_create(null, C.c_size_t(10), C.c_uint32(8), C.c_int(0), null) == 1
    assert grab.lib.grab_scan_base_window_topk(null, fake, C.c_size_t(1), C.c_uint32(1), fake, fake, fake, fake, None, None) == 1
    assert grab.lib.grab_index_scan_range_batch(null, fake, C.c_size_t(1), C.c_int(1), fake, fake, fake, fake) == 1
    assert grab.lib.grab_index_set_scan_below(null, C.c_double(0.5)) == 1


def test_oracle_is_not_linked_into_the_product():
    # the product library must not depend on the checker
    import subprocess
    out = subprocess.run(["ldd", os.path.join(ROOT, "grab-anns_amd", "libgrab_anns.so")], capture_output=True, text=True).stdout
    assert "liboracle" not in out
    src = os.path.join(ROOT, "grab-anns_amd")
    for dirpath, _, files in os.walk(src):
        for f in files:
            if f.endswith((".hip", ".cpp", ".hpp", ".py", ".h")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "oracle" not in text.lower() or f == "__init__.py" and "oracle" not in text, f
