"""CPU-only checks of the C ABI: the library loads, exports every symbol the
public header declares, and its host-only helpers agree with the oracle.  No
kernel is launched here."""
import ctypes as C
import os
import re

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "gsrast.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gs_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import gsrast_native as gn
    names = _declared()
    assert len(names) >= 26
    for n in names:
        assert hasattr(gn.lib, n), f"{n} is declared in include/gsrast.h but not exported by libgsrast.so"
    assert set(names) == set(gn.EXPORTED_SYMBOLS), set(names) ^ set(gn.EXPORTED_SYMBOLS)


def test_host_helpers(orc):
    import gsrast_native as gn
    for n in [0, 1, 2, 3, 1200, 3888, 8160, 65535, 65536, 2 ** 31]:
        assert gn.lib.gs_higher_msb(n) == orc.higher_msb(n)
    bx, by, od = C.c_int(), C.c_int(), C.c_int()
    assert gn.lib.gs_get_block_xy(C.byref(bx), C.byref(by), C.byref(od)) == 0
    assert (bx.value, by.value, od.value) == (16, 16, 256)
    assert gn.lib.gs_get_block_xy(None, None, None) != 0 and "null" in gn.last_error()


def test_state_layouts_are_aligned_and_disjoint():
    import gsrast_native as gn
    sz = [C.c_size_t() for _ in range(5)]
    assert gn.lib.gs_image_state_layout(1152, 864, *[C.byref(s) for s in sz]) == 0
    a, nc, n2, rg, tot = [s.value for s in sz]
    N = 1152 * 864
    assert a % 256 == nc % 256 == n2 % 256 == rg % 256 == 0
    assert nc >= a + 4 * N and n2 >= nc + 4 * N and rg >= n2 + 4 * N and tot >= rg + 8 * 72 * 54
    assert gn.lib.gs_binning_state_layout(1_771_093, 1152, 864, *[C.byref(s) for s in sz]) == 0
    pl, k, plu, ku, tot = [s.value for s in sz]
    R = 1_771_093
    offs = sorted([(pl, 4 * R), (k, 8 * R), (plu, 4 * R), (ku, 8 * R)])
    for (o1, l1), (o2, _) in zip(offs, offs[1:]):
        assert o1 + l1 <= o2 and o1 % 256 == 0
    assert tot > offs[-1][0] + offs[-1][1]
    assert gn.lib.gs_scan_workspace_bytes(10_000_000) >= 4 * (10_000_000 // 2048)
    assert gn.lib.gs_sort_workspace_bytes(R) >= 256 * 4 * (R // 2048)
    assert gn.lib.gs_knn_workspace_bytes(1000) > 1000 * 16


def test_layouts_and_capacities_at_the_instance_limit():
    """A view may hold up to 2^31-2 instances: at that count every array of the binning buffer still starts
    behind the one before it (no offset is formed in 32 bits), the per-instance workspaces are sized in 64 bits,
    and the radix sort over all keys, whose capacity is 2^30-2 pairs, refuses more before launching anything."""
    import gsrast_native as gn
    R = 2 ** 31 - 2
    sz = [C.c_size_t() for _ in range(5)]
    assert gn.lib.gs_binning_state_layout(R, 1920, 1080, *[C.byref(s) for s in sz]) == 0
    pl, k, plu, ku, tot = [s.value for s in sz]
    offs = sorted([(pl, 4 * R), (k, 8 * R), (plu, 4 * R), (ku, 8 * R)])
    for (o1, l1), (o2, _) in zip(offs, offs[1:]):
        assert o1 + l1 <= o2 and o1 % 256 == 0
    # point list, keys, 16-byte records, emission indices, block hits, 24 bytes of per-tile radix sort scratch
    assert tot >= (4 + 8 + 16 + 4 + 2 + 24) * R
    assert gn.lib.gs_render_backward_workspace_bytes(R) == 64 * R + 256
    assert gn.lib.gs_sort_max_pairs() == 2 ** 30 - 2
    assert gn.lib.gs_sort_workspace_bytes(2 ** 30 - 2) > 5 * 512 * 4 * ((2 ** 30 - 2) // 4096)
    one = C.c_void_p(256)  # never dereferenced: the count is refused first
    assert gn.lib.gs_sort_pairs_u64(2 ** 30 - 1, one, one, one, one, 44, one, 1 << 40, None) != 0
    assert "2^30-2" in gn.last_error()
    assert gn.lib.gs_sort_pairs_u32(2 ** 31, one, one, one, one, 32, one, 1 << 40, None) != 0
    assert "2^30-2" in gn.last_error()


def test_argument_validation_without_a_gpu():
    import gsrast_native as gn
    assert gn.lib.gs_preprocess_forward(*([None] * 8), 10, 3, 16, 0, 480, *([None] * 5), 1.0, None, None, None, 0.5, 0.5,
                                        0, 0, None, None, None) != 0
    assert "bad sizes" in gn.last_error()
    assert gn.lib.gs_sort_pairs_u64(5, None, None, None, None, 70, None, 0, None) != 0
    assert "end_bit" in gn.last_error()
    assert gn.lib.gs_mark_visible(0, None, None, None, None, None) == 0  # empty input is a no-op


def test_python_modules_refuse_cpu_tensors():
    import pytest
    import torch
    from diff_gaussian_rasterization import GaussianRasterizationSettings, GaussianRasterizer
    from simple_knn._C import distCUDA2
    rs = GaussianRasterizationSettings(32, 32, 0.5, 0.5, torch.zeros(3), 1.0, torch.eye(4), torch.eye(4), 3,
                                       torch.zeros(3), False, True, False)
    rast = GaussianRasterizer(rs)
    z = torch.zeros
    with pytest.raises(RuntimeError, match="no CPU path"):
        rast.preprocess_gaussians(z(4, 3), z(4, 3), z(4, 4), z(4, 3), z(4, 1), {})
    with pytest.raises(RuntimeError, match="no CPU path"):
        distCUDA2(z(10, 3))
