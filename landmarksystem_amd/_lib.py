"""ctypes binding of libgs355.so (the C ABI declared in include/gs355.h).

The library is built in-tree by `python -m landmarksystem_amd.csrc.build`.
There is no fallback: if the shared object is missing, loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgs355.so")

ABI_VERSION = 3  # GS355_VERSION of include/gs355.h that the structures in this file mirror

GS355_OK, GS355_EINVAL, GS355_ENOSPC, GS355_EOVERFLOW, GS355_EHIP = 0, -1, -2, -3, -4

STAGE_PREPROCESS, STAGE_SCAN, STAGE_DUPLICATE, STAGE_SORT, STAGE_RANGES, STAGE_BLEND = 1, 2, 4, 8, 16, 32
STAGE_ALL = 63
STAGE_BLEND_PLAIN = 64
STAGE_TILE_COUNT, STAGE_TILESORT, STAGE_TILE_SCATTER = 128, 256, 512
STAGE_TILE_SCATTER_TWO_LEVEL = 1024  # modifiers of STAGE_TILE_SCATTER: name the variant instead of letting the device
STAGE_TILE_SCATTER_ONE_LEVEL = 2048  # choose by the key count (which launches both)
TWO_LEVEL_MIN_KEYS = 6 << 20         # the device's own threshold
STAGE_TILESORT_SKIP = (4096, 8192, 16384)  # modifiers of STAGE_TILESORT: do not launch that size class's sorter
PIPELINE_FAST = STAGE_PREPROCESS | STAGE_TILE_COUNT | STAGE_TILE_SCATTER | STAGE_TILESORT | STAGE_BLEND
MAX_FAST_TILES = 36000 * 16  # limits of the tile-bucketed stages (the classic stages have neither)
MAX_FAST_GAUSSIANS = 1 << 28
DECODE_COUNT, DECODE_EMIT, DECODE_ALL = 1, 2, 3

EXPORTS = ("gs355_version", "gs355_last_error", "gs355_workspace_layout", "gs355_run", "gs355_render",
           "gs355_visible_filter", "gs355_anchor_filter", "gs355_decode_scratch_bytes", "gs355_decode_count",
           "gs355_decode_count_static", "gs355_decode_emit", "gs355_decode_workspace_bytes", "gs355_decode",
           "gs355_backward_scratch_bytes", "gs355_render_backward", "gs355_gather_scratch_bytes", "gs355_gather_rows")
GATHER_MAX_ARRAYS, GATHER_MAX_ROW_BYTES = 8, 4096


class Frame(C.Structure):
    _fields_ = [
        ("image_width", C.c_int32),
        ("image_height", C.c_int32),
        ("tanfovx", C.c_float),
        ("tanfovy", C.c_float),
        ("scale_modifier", C.c_float),
        ("sh_degree", C.c_int32),
        ("sh_coeffs", C.c_int32),
        ("viewmatrix", C.c_void_p),
        ("projmatrix", C.c_void_p),
        ("campos", C.c_void_p),
        ("bg", C.c_void_p),
    ]


class GatherArray(C.Structure):
    _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("row_bytes", C.c_uint32)]


class Gaussians(C.Structure):
    _fields_ = [
        ("P", C.c_int32),
        ("means3D", C.c_void_p),
        ("shs", C.c_void_p),
        ("colors_precomp", C.c_void_p),
        ("opacities", C.c_void_p),
        ("scales", C.c_void_p),
        ("rotations", C.c_void_p),
        ("cov3D_precomp", C.c_void_p),
        ("P_device", C.c_void_p),
    ]


class Outputs(C.Structure):
    _fields_ = [("image", C.c_void_p), ("depth", C.c_void_p), ("alpha", C.c_void_p), ("radii", C.c_void_p),
                ("header_copy", C.c_void_p)]


class Header(C.Structure):
    _fields_ = [
        ("num_keys_total", C.c_uint64),
        ("num_keys", C.c_uint32),
        ("overflow", C.c_uint32),
        ("num_visible", C.c_uint32),
        ("sort_class_count", C.c_uint32 * 3),
        ("reserved", C.c_uint32 * 8),
    ]


class Layout(C.Structure):
    _fields_ = [
        ("header", C.c_size_t),
        ("records", C.c_size_t),
        ("tiles_touched", C.c_size_t),
        ("rects", C.c_size_t),
        ("depth_bits", C.c_size_t),
        ("offsets", C.c_size_t),
        ("scan_tmp", C.c_size_t),
        ("keys", C.c_size_t * 2),
        ("values", C.c_size_t * 2),
        ("sort_hist", C.c_size_t),
        ("ranges", C.c_size_t),
        ("bin_matrix", C.c_size_t),
        ("tile_base", C.c_size_t),
        ("bin_visible", C.c_size_t),
        ("tile_lists", C.c_size_t),
        ("total_bytes", C.c_size_t),
        ("unsorted_buffer", C.c_int32),
        ("sorted_buffer", C.c_int32),
        ("sort_passes", C.c_int32),
        ("sort_bits", C.c_int32),
    ]


class Decoder(C.Structure):
    _fields_ = [
        ("feat_dim", C.c_int32),
        ("n_offsets", C.c_int32),
        ("in_dim", C.c_int32 * 3),
        ("w0", C.c_void_p * 3),
        ("b0", C.c_void_p * 3),
        ("w1", C.c_void_p * 3),
        ("b1", C.c_void_p * 3),
        ("add_level", C.c_int32),
        ("bank_in_dim", C.c_int32),
        ("bank_w0", C.c_void_p),
        ("bank_b0", C.c_void_p),
        ("bank_w1", C.c_void_p),
        ("bank_b1", C.c_void_p),
        ("fp32_features", C.c_int32),
        ("fp32_weights", C.c_int32),
    ]


class Anchors(C.Structure):
    _fields_ = [
        ("A", C.c_int32),
        ("anchor", C.c_void_p),
        ("feat", C.c_void_p),
        ("offset", C.c_void_p),
        ("scaling", C.c_void_p),
        ("visible_mask", C.c_void_p),
        ("campos", C.c_void_p),
        ("level", C.c_void_p),
    ]


class Decoded(C.Structure):
    _fields_ = [("xyz", C.c_void_p), ("color", C.c_void_p), ("opacity", C.c_void_p), ("scaling", C.c_void_p),
                ("rot", C.c_void_p), ("count", C.c_void_p), ("num_visible", C.c_void_p),
                ("neural_opacity", C.c_void_p), ("mask", C.c_void_p)]


class AnchorLod(C.Structure):
    _fields_ = [("level", C.c_void_p), ("extra_level", C.c_void_p), ("voxel_size", C.c_float),
                ("standard_dist", C.c_float), ("fork", C.c_float), ("resolution_scale", C.c_float),
                ("rounding", C.c_int32), ("max_level", C.c_int32)]


class BackwardInputs(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("image", "depth", "alpha", "radii", "dL_dimage", "dL_ddepth", "dL_dalpha")]


class Gradients(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("means3D", "means2D", "shs", "colors_precomp", "opacities", "scales",
                                          "rotations", "cov3D_precomp")]


class Gs355Error(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__("gs355 error %d: %s" % (code, message))
        self.code = code


_lib = None


def load() -> C.CDLL:
    """Load libgs355.so once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `python -m landmarksystem_amd.csrc.build` "
            "(there is no non-HIP fallback)" % LIB_PATH
        )
    lib = C.CDLL(LIB_PATH)
    lib.gs355_version.restype = C.c_int
    if lib.gs355_version() != ABI_VERSION:  # (the structures below would not match the library's)
        raise ImportError("%s has ABI version %d, this package binds version %d: rebuild it with "
                          "`python -m landmarksystem_amd.csrc.build`" % (LIB_PATH, lib.gs355_version(), ABI_VERSION))
    lib.gs355_last_error.restype = C.c_char_p
    lib.gs355_workspace_layout.argtypes = [C.c_int32, C.c_int64, C.c_int32, C.c_int32, C.POINTER(Layout)]
    lib.gs355_workspace_layout.restype = C.c_int
    lib.gs355_run.argtypes = [C.POINTER(Frame), C.POINTER(Gaussians), C.c_void_p, C.c_size_t, C.c_int64,
                              C.POINTER(Outputs), C.c_uint32, C.c_void_p]
    lib.gs355_run.restype = C.c_int
    lib.gs355_render.argtypes = [C.POINTER(Frame), C.POINTER(Gaussians), C.c_void_p, C.c_size_t, C.c_int64,
                                 C.POINTER(Outputs), C.c_void_p]
    lib.gs355_render.restype = C.c_int
    lib.gs355_visible_filter.argtypes = [C.POINTER(Frame), C.POINTER(Gaussians), C.c_void_p, C.c_void_p]
    lib.gs355_visible_filter.restype = C.c_int
    lib.gs355_anchor_filter.argtypes = [C.POINTER(Frame), C.POINTER(Gaussians), C.c_int32, C.POINTER(AnchorLod),
                                        C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.gs355_anchor_filter.restype = C.c_int
    lib.gs355_decode_scratch_bytes.argtypes = [C.c_int32, C.POINTER(C.c_size_t)]
    lib.gs355_decode_scratch_bytes.restype = C.c_int
    lib.gs355_decode_count.argtypes = [C.POINTER(Decoder), C.POINTER(Anchors), C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.c_size_t, C.c_void_p]
    lib.gs355_decode_count.restype = C.c_int
    lib.gs355_decode_count_static.argtypes = [C.POINTER(Decoder), C.POINTER(Anchors), C.c_void_p, C.c_void_p, C.c_void_p]
    lib.gs355_decode_count_static.restype = C.c_int
    lib.gs355_decode_emit.argtypes = [C.POINTER(Decoder), C.POINTER(Anchors), C.c_void_p, C.c_int64,
                                      C.POINTER(Decoded), C.c_void_p]
    lib.gs355_decode_emit.restype = C.c_int
    lib.gs355_decode_workspace_bytes.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_size_t)]
    lib.gs355_decode_workspace_bytes.restype = C.c_int
    lib.gs355_decode.argtypes = [C.POINTER(Decoder), C.POINTER(Anchors), C.c_int64, C.POINTER(Decoded), C.c_void_p,
                                 C.c_size_t, C.c_uint32, C.c_void_p]
    lib.gs355_decode.restype = C.c_int
    lib.gs355_backward_scratch_bytes.argtypes = [C.c_int32, C.c_int64, C.POINTER(C.c_size_t)]
    lib.gs355_backward_scratch_bytes.restype = C.c_int
    lib.gs355_render_backward.argtypes = [C.POINTER(Frame), C.POINTER(Gaussians), C.c_void_p, C.c_size_t, C.c_int64,
                                          C.POINTER(BackwardInputs), C.c_void_p, C.c_size_t, C.POINTER(Gradients),
                                          C.c_void_p]
    lib.gs355_render_backward.restype = C.c_int
    lib.gs355_gather_scratch_bytes.argtypes = [C.c_int32, C.POINTER(C.c_size_t)]
    lib.gs355_gather_scratch_bytes.restype = C.c_int
    lib.gs355_gather_rows.argtypes = [C.c_int32, C.c_void_p, C.c_int32, C.POINTER(GatherArray), C.c_void_p, C.c_void_p,
                                      C.c_size_t, C.c_void_p]
    lib.gs355_gather_rows.restype = C.c_int
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != GS355_OK:
        raise Gs355Error(rc, load().gs355_last_error().decode("utf-8", "replace"))


def workspace_layout(P: int, n_cap: int, width: int, height: int) -> Layout:
    L = Layout()
    check(load().gs355_workspace_layout(int(P), int(n_cap), int(width), int(height), C.byref(L)))
    return L
