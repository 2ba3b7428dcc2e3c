"""ctypes binding of libgsrast.so (C ABI declared in include/gsrast.h).

There is no fallback: if the library is missing or a symbol cannot be
resolved, importing this module raises, and every entry point raises
RuntimeError with the library's message on a non-zero status.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libgsrast.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} not found: build it first (make -C {os.path.join(_HERE, 'csrc')} "
        "or __graft_entry__.build()); there is no CPU fallback")

lib = C.CDLL(LIB_PATH)

RESIZE_FN = C.CFUNCTYPE(C.c_void_p, C.c_size_t, C.c_void_p)

_vp, _i, _f, _sz, _i64 = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_int64
_psz = C.POINTER(C.c_size_t)

_SIGNATURES = {
    "gs_last_error": (C.c_char_p, []),
    "gs_get_block_xy": (_i, [C.POINTER(_i)] * 3),
    "gs_higher_msb": (C.c_uint32, [C.c_uint32]),
    "gs_mark_visible": (_i, [_i, _vp, _vp, _vp, _vp, _vp]),
    "gs_visible_filter": (_i, [_i, _i, _i, _i, _vp, _vp, _f, _vp, _vp, _vp, _vp, _f, _f, _i, _vp, _i, _vp]),
    "gs_preprocess_forward": (_i, [_vp] * 8 + [_i] * 5 + [_vp] * 5 + [_f] + [_vp] * 3 + [_f, _f, _i, _i, _vp, _vp,
                                   _vp]),
    "gs_preprocess_backward": (_i, [_vp] * 3 + [_i] * 5 + [_vp] * 4 + [_f] + [_vp] * 3 + [_f, _f] + [_vp, _i] +
                               [_vp] * 8 + [_i, _vp, _vp]),
    "gs_render_forward": (_i, [RESIZE_FN, _vp, RESIZE_FN, _vp, RESIZE_FN, _vp, _i, _vp, _i, _i, _f, _f, _f, _f] +
                          [_vp] * 17 + [_i, _i, C.POINTER(_i), C.POINTER(_f), _vp, _vp, _vp]),
    "gs_render_backward_workspace_bytes": (_sz, [_i]),
    "gs_render_backward": (_i, [_i, _i, _vp, _i, _i, _f, _f] + [_vp] * 17 + [_i, _i, _vp, _sz, C.POINTER(_f), _i64,
                                _vp, _vp]),
    "gs_ssim_l1_forward": (_i, [_i, _i, _i] + [_vp] * 9),
    "gs_ssim_l1_backward": (_i, [_i, _i, _i] + [_vp] * 10),
    "gs_training_stats_workspace_bytes": (_sz, [_i64, _i64]),
    "gs_training_stats": (_i, [_i64, _i, _i64, _i64, _vp, _vp, _vp, _vp, _i] + [_vp] * 6 + [_sz, _vp]),
    "gs_max_radii_update": (_i, [_i64, _vp, _vp, _vp, _vp]),
    "gs_adam_step": (_i, [_i] + [_vp] * 7 + [C.c_double, C.c_double, C.c_double, _f, _vp]),
    "gs_neural_supported": (_i, [_i]),
    "gs_neural_workspace_bytes": (_sz, [_i64, _i]),
    "gs_neural_opacity_forward": (_i, [_i64, _i] + [_vp] * 6 + [_i] + [_vp] * 5 + [_sz, _vp, _vp]),
    "gs_neural_gaussians_forward": (_i, [_i64, _i, _i64] + [_vp] * 9 + [_sz] + [_vp] * 7),
    "gs_neural_backward_workspace_bytes": (_sz, [_i64, _i]),
    "gs_neural_backward": (_i, [_i64, _i, _i64] + [_vp] * 8 + [_i] + [_vp] * 17 + [_sz, _vp]),
    "gs_all_map_forward": (_i, [_i] + [_vp] * 7),
    "gs_all_map_backward": (_i, [_i] + [_vp] * 9),
    "gs_knn_workspace_bytes": (_sz, [_i]),
    "gs_knn_dist2": (_i, [_i, _vp, _vp, _vp, _sz, _vp]),
    "gs_tile_count": (_i, [_i, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "gs_scan_workspace_bytes": (_sz, [_i64]),
    "gs_inclusive_sum": (_i, [_i64, _vp, _vp, _vp, _sz, _vp]),
    "gs_inclusive_sum_static_max": (_i64, []),
    "gs_inclusive_sum_static": (_i, [_i64, _vp, _vp, _vp]),
    "gs_duplicate_with_keys": (_i, [_i, _i, _i] + [_vp] * 8),
    "gs_sort_workspace_bytes": (_sz, [_i64]),
    "gs_sort_max_pairs": (_i64, []),
    "gs_sort_status": (_i, [_vp, _vp]),
    "gs_sort_workspace_error_offset": (_sz, []),
    "gs_sort_check_async": (_i, [_vp, _vp]),
    "gs_pending_fault": (_i, []),
    "gs_sort_pairs_u64": (_i, [_i64, _vp, _vp, _vp, _vp, _i, _vp, _sz, _vp]),
    "gs_sort_pairs_u32": (_i, [_i64, _vp, _vp, _vp, _vp, _i, _vp, _sz, _vp]),
    "gs_identify_tile_ranges": (_i, [_i64, _vp, _i, _vp, _vp]),
    "gs_render_tiles_forward": (_i, [_i, _i, _i, _f, _f, _f, _f] + [_vp] * 8 + [_i] + [_vp] * 11),
    "gs_render_tiles_backward": (_i, [_i, _i, _i, _f, _f] + [_vp] * 14 + [_i] + [_vp] * 9),
    "gs_selftest_reductions": (_i, [_vp, _vp, _vp, _vp]),
    "gs_stage_timing_enable": (_i, [_i]),
    "gs_stage_timing_collect": (_i, [C.c_char_p, _sz]),
    "gs_image_state_layout": (_i, [_i, _i] + [_psz] * 5),
    "gs_binning_state_layout": (_i, [_i64, _i, _i] + [_psz] * 5),
    "gs_geometry_state_layout": (_i, [_i] + [_psz] * 3),
}

for _name, (_res, _args) in _SIGNATURES.items():
    _fn = getattr(lib, _name)  # AttributeError here = the library lacks a declared symbol
    _fn.restype = _res
    _fn.argtypes = _args

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


class RenderOptions(C.Structure):
    """gs_render_options of include/gsrast.h; a negative limit keeps the library's default, a zero expectation
    means none."""
    _fields_ = [("struct_bytes", C.c_uint32), ("tile_sort_small_limit", C.c_int32),
                ("tile_sort_block_records", C.c_int32), ("expected_longest_list", C.c_int32),
                ("expected_instances", C.c_int64), ("blend_records", C.c_void_p)]

    def __init__(self, tile_sort_small_limit=-1, tile_sort_block_records=-1, expected_instances=0,
                 expected_longest_list=0, blend_records=None):
        super().__init__(C.sizeof(RenderOptions), int(tile_sort_small_limit), int(tile_sort_block_records),
                         int(expected_longest_list), int(expected_instances), blend_records)


class RenderResult(C.Structure):
    """gs_render_result of include/gsrast.h."""
    _fields_ = [("struct_bytes", C.c_uint32), ("longest_list", C.c_int32), ("binning_capacity", C.c_int64),
                ("launched_ahead", C.c_int32), ("reserved", C.c_int32)]

    def __init__(self):
        super().__init__(C.sizeof(RenderResult), 0, 0, 0, 0)


def stage_timing(enable):
    check(lib.gs_stage_timing_enable(int(bool(enable))), "gs_stage_timing_enable")


def stage_timing_collect():
    """{stage: (total_ms, launches)} since the last collect."""
    buf = C.create_string_buffer(8192)
    check(lib.gs_stage_timing_collect(buf, len(buf)), "gs_stage_timing_collect")
    out = {}
    for line in buf.value.decode().splitlines():
        name, ms, cnt = line.split()
        out[name] = (float(ms), int(cnt))
    return out


def last_error():
    return lib.gs_last_error().decode("utf-8", "replace")


def check(status, what):
    if status != 0:
        raise RuntimeError(f"{what}: {last_error()}")
