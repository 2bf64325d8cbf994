"""Host side of the C ABI, no GPU needed: the library loads, exports exactly the
symbols include/gs355.h declares, lays the workspace out sanely and rejects bad
arguments before touching HIP."""
import ctypes as C
import os
import re

import pytest

from landmarksystem_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "gs355.h")).read()
    return sorted(set(re.findall(r"GS355_API\s+[\w\s\*]+?\b(gs355_\w+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_functions()
    assert names == sorted(_lib.EXPORTS)
    for n in names:
        assert hasattr(lib, n), n
    assert lib.gs355_version() == _lib.ABI_VERSION == 3


def test_struct_sizes_match_the_header():
    # 64-byte header; pointers are 8 bytes; the layout struct mirrors include/gs355.h field by field
    assert C.sizeof(_lib.Header) == 64
    assert C.sizeof(_lib.Frame) == 7 * 4 + 4 + 4 * 8  # 7 scalars, padding to 8, 4 pointers
    assert C.sizeof(_lib.Gaussians) == 8 + 8 * 8  # P (padded to 8), 7 tensors, the optional device-side count
    assert C.sizeof(_lib.Outputs) == 5 * 8  # image, depth, alpha, radii, the optional second copy of the header
    assert C.sizeof(_lib.Layout) == 18 * 8 + 4 * 4
    assert C.sizeof(_lib.AnchorLod) == 2 * 8 + 4 * 4 + 2 * 4
    assert C.sizeof(_lib.BackwardInputs) == 7 * 8 and C.sizeof(_lib.Gradients) == 8 * 8


def test_workspace_layout_is_aligned_ordered_and_sized():
    P, n_cap, W, H = 100_000, 1_500_000, 1920, 1080
    L = _lib.workspace_layout(P, n_cap, W, H)
    offs = [L.header, L.records, L.tiles_touched, L.rects, L.depth_bits, L.offsets, L.scan_tmp, L.keys[0], L.keys[1], L.values[0],
            L.values[1], L.sort_hist, L.ranges, L.bin_matrix, L.tile_base, L.bin_visible, L.tile_lists, L.total_bytes]
    assert all(o % 256 == 0 for o in offs)
    assert offs == sorted(offs) and len(set(offs)) == len(offs)
    assert L.records - L.header >= 64
    assert L.tiles_touched - L.records >= P * 48 and L.depth_bits - L.rects >= P * 8
    assert L.keys[1] - L.keys[0] >= n_cap * 8
    assert L.values[1] - L.values[0] >= n_cap * 4
    tiles = 120 * 68
    assert L.bin_matrix - L.ranges >= tiles * 8 and L.total_bytes - L.tile_lists >= (4 + 4 * tiles) * 4
    assert L.tile_base - L.bin_matrix >= 256 * tiles * 4
    assert L.bin_visible - L.tile_base >= 2 * tiles * 4  # bases, then the scatter's cursors
    # beyond 36000 tiles the slices count per coarse bin of 16 tiles
    Lw = _lib.workspace_layout(10, 10, 7680, 4320)
    wide_tiles = 480 * 270
    assert 256 * (wide_tiles // 16) * 4 <= Lw.tile_base - Lw.bin_matrix < 256 * (wide_tiles // 16) * 4 + 256
    assert L.sort_bits == 32 + 13 and L.sort_passes == 6 and L.sorted_buffer == 0
    L4k = _lib.workspace_layout(10, 10, 3840, 2160)
    assert L4k.sort_bits == 47 and L4k.sort_passes == 6
    Ls = _lib.workspace_layout(10, 10, 256, 256)  # 256 tiles -> 40 bits -> 5 passes -> result in buffer 1
    assert Ls.sort_bits == 40 and Ls.sort_passes == 5 and Ls.sorted_buffer == 1
    L0 = _lib.workspace_layout(0, 0, 16, 16)
    assert L0.total_bytes > 0


def _err(code_expected, fn, *args):
    rc = fn(*args)
    assert rc == code_expected, (rc, _lib.load().gs355_last_error())
    return _lib.load().gs355_last_error().decode()


def test_layout_rejects_bad_dimensions():
    lib = _lib.load()
    L = _lib.Layout()
    assert "P must be" in _err(_lib.GS355_EINVAL, lib.gs355_workspace_layout, -1, 10, 64, 64, C.byref(L))
    assert "image size" in _err(_lib.GS355_EINVAL, lib.gs355_workspace_layout, 1, 10, 0, 64, C.byref(L))
    assert "n_cap" in _err(_lib.GS355_EINVAL, lib.gs355_workspace_layout, 1, -5, 64, 64, C.byref(L))
    assert "32-bit" in _err(_lib.GS355_EOVERFLOW, lib.gs355_workspace_layout, 1, 1 << 32, 64, 64, C.byref(L))
    assert "tiles" in _err(_lib.GS355_EOVERFLOW, lib.gs355_workspace_layout, 1, 10, 1 << 20, 1 << 20, C.byref(L))
    assert _err(_lib.GS355_EINVAL, lib.gs355_workspace_layout, 1, 10, 64, 64, None)
    with pytest.raises(_lib.Gs355Error) as e:
        _lib.workspace_layout(-3, 0, 8, 8)
    assert e.value.code == _lib.GS355_EINVAL


def _frame(W=64, H=64, deg=0, coeffs=1, ptr=0x1000):
    f = _lib.Frame()
    f.image_width, f.image_height, f.tanfovx, f.tanfovy, f.scale_modifier = W, H, 0.5, 0.5, 1.0
    f.sh_degree, f.sh_coeffs = deg, coeffs
    f.viewmatrix = f.projmatrix = f.campos = f.bg = ptr
    return f


def _gauss(P=10, shs=True, colors=False, sr=True, cov=False, ptr=0x1000):
    g = _lib.Gaussians()
    g.P = P
    g.means3D = g.opacities = ptr
    g.shs = ptr if shs else None
    g.colors_precomp = ptr if colors else None
    g.scales = g.rotations = (ptr if sr else None)
    g.cov3D_precomp = ptr if cov else None
    return g


def test_run_validates_before_any_hip_call():
    """All of these return before a kernel could be launched: the fake
    pointers are never dereferenced and no GPU is needed."""
    lib = _lib.load()
    out = _lib.Outputs()
    out.image = out.radii = 0x1000
    run = lambda f, g, ws, nbytes, cap, o, mask: lib.gs355_run(  # noqa: E731
        C.byref(f) if f else None, C.byref(g) if g else None, ws, nbytes, cap, C.byref(o) if o else None, mask, None)
    f, g = _frame(), _gauss()
    assert "frame is NULL" in _err(_lib.GS355_EINVAL, run, None, g, 0x1000, 1 << 30, 100, out, _lib.STAGE_ALL)
    assert "gaussians is NULL" in _err(_lib.GS355_EINVAL, run, f, None, 0x1000, 1 << 30, 100, out, _lib.STAGE_ALL)
    assert "stage_mask" in _err(_lib.GS355_EINVAL, run, f, g, 0x1000, 1 << 30, 100, out, 0)
    assert "stage_mask" in _err(_lib.GS355_EINVAL, run, f, g, 0x1000, 1 << 30, 100, out, 1024)  # a modifier alone
    assert "stage_mask" in _err(_lib.GS355_EINVAL, run, f, g, 0x1000, 1 << 30, 100, out, 2048)
    assert "stage_mask" in _err(_lib.GS355_EINVAL, run, f, g, 0x1000, 1 << 30, 100, out, _lib.PIPELINE_FAST | 1024 | 2048)
    assert "stage_mask" in _err(_lib.GS355_EINVAL, run, f, g, 0x1000, 1 << 30, 100, out, sum(_lib.STAGE_TILESORT_SKIP))
    assert "stage_mask" in _err(_lib.GS355_EINVAL, run, f, g, 0x1000, 1 << 30, 100, out, 32768)  # no such stage
    assert "SHs or precomputed colors" in _err(_lib.GS355_EINVAL, run, f, _gauss(shs=True, colors=True), 0x1000,
                                                1 << 30, 100, out, _lib.STAGE_ALL)
    assert "SHs or precomputed colors" in _err(_lib.GS355_EINVAL, run, f, _gauss(shs=False, colors=False), 0x1000,
                                                1 << 30, 100, out, _lib.STAGE_ALL)
    assert "scale/rotation" in _err(_lib.GS355_EINVAL, run, f, _gauss(sr=True, cov=True), 0x1000, 1 << 30, 100, out,
                                     _lib.STAGE_ALL)
    assert "scale/rotation" in _err(_lib.GS355_EINVAL, run, f, _gauss(sr=False, cov=False), 0x1000, 1 << 30, 100,
                                     out, _lib.STAGE_ALL)
    assert "sh_degree" in _err(_lib.GS355_EINVAL, run, _frame(deg=4, coeffs=25), g, 0x1000, 1 << 30, 100, out,
                               _lib.STAGE_ALL)
    assert "coefficients" in _err(_lib.GS355_EINVAL, run, _frame(deg=3, coeffs=4), g, 0x1000, 1 << 30, 100, out,
                                  _lib.STAGE_ALL)
    bad = _frame()
    bad.tanfovx = 0.0
    assert "tanfov" in _err(_lib.GS355_EINVAL, run, bad, g, 0x1000, 1 << 30, 100, out, _lib.STAGE_ALL)
    assert "workspace is NULL" in _err(_lib.GS355_EINVAL, run, f, g, None, 1 << 30, 100, out, _lib.STAGE_ALL)
    assert "aligned" in _err(_lib.GS355_EINVAL, run, f, g, 0x1001, 1 << 30, 100, out, _lib.STAGE_ALL)
    msg = _err(_lib.GS355_ENOSPC, run, f, g, 0x1000, 1024, 100, out, _lib.STAGE_ALL)
    assert "needed" in msg
    assert "32-bit" in _err(_lib.GS355_EOVERFLOW, run, f, g, 0x1000, 1 << 30, 1 << 33, out, _lib.STAGE_ALL)
    # limits of the tile-bucketed stages: 576000 tiles (16 x 36000), 2^28 Gaussians; the classic stages have neither
    wide = _frame(W=16 * 1000, H=16 * 577)
    assert "at most 576000 tiles" in _err(_lib.GS355_EINVAL, run, wide, g, 0x1000, 1 << 30, 100, out, _lib.PIPELINE_FAST)
    assert "needed" in _err(_lib.GS355_ENOSPC, run, wide, g, 0x1000, 1024, 100, out, _lib.STAGE_ALL)
    assert "Gaussians; use the classic" in _err(_lib.GS355_EINVAL, run, f, _gauss(P=(1 << 28) + 1), 0x1000, 1 << 30, 100,
                                                 out, _lib.PIPELINE_FAST)
    no_img = _lib.Outputs()
    no_img.radii = 0x1000
    assert "image is NULL" in _err(_lib.GS355_EINVAL, run, f, g, 0x1000, 1 << 30, 100, no_img, _lib.STAGE_BLEND)
    no_radii = _lib.Outputs()
    no_radii.image = 0x1000
    assert "radii is NULL" in _err(_lib.GS355_EINVAL, run, f, g, 0x1000, 1 << 30, 100, no_radii, _lib.STAGE_ALL)


def test_render_backward_validates_before_any_hip_call():
    lib = _lib.load()
    size = C.c_size_t(0)
    assert lib.gs355_backward_scratch_bytes(1000, 5000, C.byref(size)) == 0
    assert size.value >= 5000 * 48 + 1000 * 4 and size.value % 256 == 0
    assert "P must be" in _err(_lib.GS355_EINVAL, lib.gs355_backward_scratch_bytes, -1, 10, C.byref(size))
    assert "n_cap" in _err(_lib.GS355_EINVAL, lib.gs355_backward_scratch_bytes, 10, -1, C.byref(size))
    assert _err(_lib.GS355_EINVAL, lib.gs355_backward_scratch_bytes, 10, 10, None)

    def bwd(f, g, ws, nbytes, cap, b, scratch, sbytes, grads):
        return lib.gs355_render_backward(C.byref(f) if f else None, C.byref(g) if g else None, ws, nbytes, cap,
                                         C.byref(b) if b else None, scratch, sbytes, C.byref(grads) if grads else None,
                                         None)

    f, g = _frame(), _gauss()
    b = _lib.BackwardInputs(0x1000, None, None, 0x1000, 0x1000, None, None)
    grads = _lib.Gradients()
    grads.means3D = 0x1000
    ok = (f, g, 0x1000, 1 << 30, 100, b, 0x1000, 1 << 20, grads)

    def with_(**kw):
        names = ("f", "g", "ws", "nbytes", "cap", "b", "scratch", "sbytes", "grads")
        args = dict(zip(names, ok))
        args.update(kw)
        return [args[n] for n in names]

    assert "frame is NULL" in _err(_lib.GS355_EINVAL, bwd, *with_(f=None))
    assert "gaussians is NULL" in _err(_lib.GS355_EINVAL, bwd, *with_(g=None))
    assert "backward inputs is NULL" in _err(_lib.GS355_EINVAL, bwd, *with_(b=None))
    assert "gradients is NULL" in _err(_lib.GS355_EINVAL, bwd, *with_(grads=None))
    assert "dL_dimage" in _err(_lib.GS355_EINVAL, bwd, *with_(b=_lib.BackwardInputs(0x1000, None, None, 0x1000, None, None, None)))
    assert "forward depth" in _err(_lib.GS355_EINVAL, bwd, *with_(b=_lib.BackwardInputs(0x1000, None, None, 0x1000, 0x1000, 0x1000, None)))
    assert "forward alpha" in _err(_lib.GS355_EINVAL, bwd, *with_(b=_lib.BackwardInputs(0x1000, None, None, 0x1000, 0x1000, None, 0x1000)))
    assert "radii is NULL" in _err(_lib.GS355_EINVAL, bwd, *with_(b=_lib.BackwardInputs(0x1000, None, None, None, 0x1000, None, None)))
    wrong = _lib.Gradients()
    wrong.colors_precomp = 0x1000  # the frame was rendered from SH coefficients
    assert "not given" in _err(_lib.GS355_EINVAL, bwd, *with_(grads=wrong))
    assert "SHs or precomputed colors" in _err(_lib.GS355_EINVAL, bwd, *with_(g=_gauss(shs=True, colors=True)))
    assert "workspace is NULL" in _err(_lib.GS355_EINVAL, bwd, *with_(ws=None))
    assert "aligned" in _err(_lib.GS355_EINVAL, bwd, *with_(ws=0x1001))
    assert "needed" in _err(_lib.GS355_ENOSPC, bwd, *with_(nbytes=1024))
    assert "scratch is NULL" in _err(_lib.GS355_EINVAL, bwd, *with_(scratch=None))
    assert "256-byte" in _err(_lib.GS355_EINVAL, bwd, *with_(scratch=0x1004))
    assert "scratch has" in _err(_lib.GS355_ENOSPC, bwd, *with_(sbytes=16))
    assert "32-bit" in _err(_lib.GS355_EOVERFLOW, bwd, *with_(cap=1 << 33))


def test_visible_filter_validates():
    lib = _lib.load()
    f, g = _frame(), _gauss(shs=False)
    vf = lambda f, g, r: lib.gs355_visible_filter(C.byref(f) if f else None, C.byref(g) if g else None, r, None)  # noqa: E731
    assert "frame is NULL" in _err(_lib.GS355_EINVAL, vf, None, g, 0x1000)
    assert "radii is NULL" in _err(_lib.GS355_EINVAL, vf, f, g, None)
    assert "scale/rotation" in _err(_lib.GS355_EINVAL, vf, f, _gauss(sr=False), 0x1000)
    half = _gauss()
    half.rotations = None
    assert "scale/rotation" in _err(_lib.GS355_EINVAL, vf, f, half, 0x1000)


def test_anchor_filter_validates_before_any_hip_call():
    lib = _lib.load()
    f, g = _frame(), _gauss(shs=False)

    def af(f, g, stride, lod, visible):
        return lib.gs355_anchor_filter(C.byref(f) if f else None, C.byref(g) if g else None, stride,
                                       C.byref(lod) if lod else None, None, visible, None, None)

    lod = _lib.AnchorLod(0x1000, 0x1000, 0.5, 250.0, 2.0, 1.0, 1, 4)
    assert "frame is NULL" in _err(_lib.GS355_EINVAL, af, None, g, 6, None, 0x1000)
    assert "visible is NULL" in _err(_lib.GS355_EINVAL, af, f, g, 6, None, None)
    assert "scale_stride" in _err(_lib.GS355_EINVAL, af, f, g, 2, None, 0x1000)
    assert "scale/rotation" in _err(_lib.GS355_EINVAL, af, f, _gauss(sr=False), 6, None, 0x1000)
    bad = _lib.AnchorLod(0x1000, None, 0.5, 250.0, 2.0, 1.0, 1, 4)
    assert "extra_level is NULL" in _err(_lib.GS355_EINVAL, af, f, g, 6, bad, 0x1000)
    bad = _lib.AnchorLod(0x1000, 0x1000, 0.5, 250.0, 2.0, 1.0, 3, 4)
    assert "rounding" in _err(_lib.GS355_EINVAL, af, f, g, 6, bad, 0x1000)
    bad = _lib.AnchorLod(0x1000, 0x1000, 0.5, 250.0, 1.0, 1.0, 1, 4)
    assert "fork must be > 1" in _err(_lib.GS355_EINVAL, af, f, g, 6, bad, 0x1000)
    no_cam = _frame()
    no_cam.campos = None
    assert "campos" in _err(_lib.GS355_EINVAL, af, no_cam, g, 6, lod, 0x1000)
    empty = _gauss(shs=False)
    empty.P = 0
    assert af(f, empty, 6, lod, None) == 0  # nothing to do, nothing launched


def _decoder(feat=32, n=10, in_dim=(36, 36, 36), ptr=0x1000):
    d = _lib.Decoder()
    d.feat_dim, d.n_offsets = feat, n
    for j in range(3):
        d.in_dim[j] = in_dim[j]
        d.w0[j] = d.b0[j] = d.w1[j] = d.b1[j] = ptr
    return d


def _anchors(A=10, ptr=0x1000):
    a = _lib.Anchors()
    a.A = A
    a.anchor = a.feat = a.offset = a.scaling = a.visible_mask = a.campos = ptr
    return a


def test_decode_validates_before_any_hip_call():
    lib = _lib.load()
    count = lambda d, a, c, o, s, n: lib.gs355_decode_count(C.byref(d), C.byref(a), c, o, s, n, None)  # noqa: E731
    assert "feat_dim" in _err(_lib.GS355_EINVAL, count, _decoder(feat=64), _anchors(), 0x1000, 0x1000, 0x1000, 1 << 20)
    assert "offsets per anchor" in _err(_lib.GS355_EINVAL, count, _decoder(n=11), _anchors(), 0x1000, 0x1000, 0x1000,
                                        1 << 20)
    assert "input width" in _err(_lib.GS355_EINVAL, count, _decoder(in_dim=(36, 40, 36)), _anchors(), 0x1000, 0x1000,
                                 0x1000, 1 << 20)
    bad = _decoder()
    bad.w1[2] = None
    assert "head 2" in _err(_lib.GS355_EINVAL, count, bad, _anchors(), 0x1000, 0x1000, 0x1000, 1 << 20)
    missing = _anchors()
    missing.offset = None
    assert "non-NULL" in _err(_lib.GS355_EINVAL, count, _decoder(), missing, 0x1000, 0x1000, 0x1000, 1 << 20)
    assert "aligned" in _err(_lib.GS355_EINVAL, count, _decoder(), _anchors(ptr=0x1004), 0x1000, 0x1000, 0x1000, 1 << 20)
    assert "scratch" in _err(_lib.GS355_EINVAL, count, _decoder(), _anchors(), 0x1000, 0x1000, None, 1 << 20)
    assert "needed" in _err(_lib.GS355_ENOSPC, count, _decoder(), _anchors(A=100_000), 0x1000, 0x1000, 0x1000, 16)
    out = _lib.Decoded()
    emit = lambda d, a, o, cap, dst: lib.gs355_decode_emit(C.byref(d), C.byref(a), o, cap, C.byref(dst), None)  # noqa: E731
    assert "outputs" in _err(_lib.GS355_EINVAL, emit, _decoder(), _anchors(), 0x1000, 10, out)
    assert "capacity" in _err(_lib.GS355_EINVAL, emit, _decoder(), _anchors(), 0x1000, -1, out)
    need = C.c_size_t()
    assert lib.gs355_decode_scratch_bytes(1000, C.byref(need)) == 0 and need.value >= 256


def test_one_call_decode_validates_before_any_hip_call():
    """gs355_decode / gs355_decode_workspace_bytes: phases, capacity, outputs, workspace, feature bank and level
    input are all checked before anything could be launched."""
    lib = _lib.load()
    out = _lib.Decoded()

    def dec(d, a, cap, o, ws, nbytes, phases):
        return lib.gs355_decode(C.byref(d), C.byref(a), cap, C.byref(o) if o is not None else None, ws, nbytes, phases, None)

    ok = (_decoder(), _anchors(), 100, out, 0x1000, 1 << 30)
    assert "phases" in _err(_lib.GS355_EINVAL, dec, *ok, 0)
    assert "phases" in _err(_lib.GS355_EINVAL, dec, *ok, 4)
    assert "feat_dim" in _err(_lib.GS355_EINVAL, dec, _decoder(feat=64), *ok[1:], _lib.DECODE_ALL)
    assert "capacity" in _err(_lib.GS355_EINVAL, dec, _decoder(), _anchors(), -1, out, 0x1000, 1 << 30, _lib.DECODE_ALL)
    assert "capacity" in _err(_lib.GS355_EINVAL, dec, _decoder(), _anchors(), 1 << 32, out, 0x1000, 1 << 30, _lib.DECODE_ALL)
    assert "outputs is NULL" in _err(_lib.GS355_EINVAL, dec, _decoder(), _anchors(), 100, None, 0x1000, 1 << 30,
                                     _lib.DECODE_ALL)
    assert "non-NULL" in _err(_lib.GS355_EINVAL, dec, *ok, _lib.DECODE_EMIT)  # the five output arrays are missing
    assert "workspace is NULL" in _err(_lib.GS355_EINVAL, dec, _decoder(), _anchors(), 100, out, None, 1 << 30,
                                       _lib.DECODE_COUNT)
    assert "aligned" in _err(_lib.GS355_EINVAL, dec, _decoder(), _anchors(), 100, out, 0x1010, 1 << 30, _lib.DECODE_COUNT)
    assert "needed" in _err(_lib.GS355_ENOSPC, dec, _decoder(), _anchors(A=100_000), 100, out, 0x1000, 64,
                            _lib.DECODE_COUNT)
    # level input: every head reads [feat | view | level] (36 columns) and the level array must be there
    lvl = _decoder(in_dim=(36, 36, 36))
    lvl.add_level = 1
    assert "level" in _err(_lib.GS355_EINVAL, dec, lvl, _anchors(), 100, out, 0x1000, 1 << 30, _lib.DECODE_COUNT)
    narrow = _decoder(in_dim=(35, 35, 35))
    narrow.add_level = 1
    an = _anchors()
    an.level = 0x1000
    assert _err(_lib.GS355_EINVAL, dec, narrow, an, 100, out, 0x1000, 1 << 30, _lib.DECODE_COUNT)
    # feature bank: its input is [view] or [view | level], and all four weight arrays must be given
    bank = _decoder()
    bank.bank_in_dim = 5
    assert "bank" in _err(_lib.GS355_EINVAL, dec, bank, _anchors(), 100, out, 0x1000, 1 << 30, _lib.DECODE_COUNT)
    bank.bank_in_dim = 3
    assert "bank" in _err(_lib.GS355_EINVAL, dec, bank, _anchors(), 100, out, 0x1000, 1 << 30, _lib.DECODE_COUNT)
    # the two-call entry points have no workspace for the mixed features
    bank.bank_w0 = bank.bank_b0 = bank.bank_w1 = bank.bank_b1 = 0x1000
    assert "bank" in _err(_lib.GS355_EINVAL, lib.gs355_decode_count, C.byref(bank), C.byref(_anchors()), 0x1000, 0x1000,
                          0x1000, 1 << 20, None)

    need, with_bank = C.c_size_t(), C.c_size_t()
    assert lib.gs355_decode_workspace_bytes(500_000, 10, 0, C.byref(need)) == 0
    assert lib.gs355_decode_workspace_bytes(500_000, 10, 1, C.byref(with_bank)) == 0
    assert need.value % 256 == 0 and with_bank.value >= need.value + 500_000 * 32 * 4
    assert "offsets per anchor" in _err(_lib.GS355_EINVAL, lib.gs355_decode_workspace_bytes, 10, 11, 0, C.byref(need))
    assert "A must be" in _err(_lib.GS355_EINVAL, lib.gs355_decode_workspace_bytes, -1, 10, 0, C.byref(need))
    assert _err(_lib.GS355_EINVAL, lib.gs355_decode_workspace_bytes, 10, 10, 0, None)


def test_gather_rows_validates_before_hip():
    lib = _lib.load()
    need = C.c_size_t()
    assert lib.gs355_gather_scratch_bytes(6_000_000, C.byref(need)) == 0 and 8 * 5860 <= need.value < 1 << 20
    assert "P must be" in _err(_lib.GS355_EINVAL, lib.gs355_gather_scratch_bytes, -1, C.byref(need))
    arrays = (_lib.GatherArray * 2)()
    arrays[0].src, arrays[0].dst, arrays[0].row_bytes = 0x1000, 0x2000, 12
    arrays[1].src, arrays[1].dst, arrays[1].row_bytes = 0x1000, 0x2000, 192
    call = lambda *a: _err(_lib.GS355_EINVAL, lib.gs355_gather_rows, *a)  # noqa: E731
    assert "n_arrays" in call(10, 0x1000, 9, arrays, None, 0x1000, 1 << 20, None)
    assert "mask is NULL" in call(10, None, 2, arrays, None, 0x1000, 1 << 20, None)
    assert "scratch is NULL" in call(10, 0x1000, 2, arrays, None, None, 1 << 20, None)
    arrays[1].row_bytes = 194
    assert "multiple of 4" in call(10, 0x1000, 2, arrays, None, 0x1000, 1 << 20, None)
    arrays[1].row_bytes = 8192
    assert "multiple of 4" in call(10, 0x1000, 2, arrays, None, 0x1000, 1 << 20, None)
    arrays[1].row_bytes, arrays[1].dst = 192, None
    assert "src / dst is NULL" in call(10, 0x1000, 2, arrays, None, 0x1000, 1 << 20, None)
    arrays[1].dst = 0x2002
    assert "aligned" in call(10, 0x1000, 2, arrays, None, 0x1000, 1 << 20, None)
    arrays[1].dst = 0x2000
    assert "too small" in _err(_lib.GS355_ENOSPC, lib.gs355_gather_rows, 10_000, 0x1000, 2, arrays, None, 0x1000, 16, None)


def test_header_is_plain_c(tmp_path):
    """include/gs355.h must compile as C99 (the boundary carries no C++ or torch types), and a C caller's view of the
    struct sizes must match what the Python binding assumes."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "probe.c"
    src.write_text(
        '#include <stdio.h>\n#include "gs355.h"\n'
        "int main(void) {\n"
        '  printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu\\n", sizeof(gs355_header), sizeof(gs355_frame),\n'
        "         sizeof(gs355_gaussians), sizeof(gs355_outputs), sizeof(gs355_layout), sizeof(gs355_anchor_lod),\n"
        "         sizeof(gs355_decoder), sizeof(gs355_anchors), sizeof(gs355_decoded));\n"
        "  return GS355_PIPELINE_FAST == (GS355_STAGE_PREPROCESS | GS355_STAGE_TILE_COUNT | GS355_STAGE_TILE_SCATTER |\n"
        "                                 GS355_STAGE_TILESORT | GS355_STAGE_BLEND) ? 0 : 1;\n}\n")
    exe = tmp_path / "probe"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(root, "include"), str(src),
                    "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    want = [C.sizeof(t) for t in (_lib.Header, _lib.Frame, _lib.Gaussians, _lib.Outputs, _lib.Layout, _lib.AnchorLod,
                                  _lib.Decoder, _lib.Anchors, _lib.Decoded)]
    assert [int(v) for v in out] == want


def test_static_count_rejects_more_anchors_than_its_array_covers():
    lib = _lib.load()
    d = _lib.Decoder()
    d.feat_dim, d.n_offsets = 32, 10
    for j in range(3):
        d.in_dim[j] = 36
        d.w0[j] = d.b0[j] = d.w1[j] = d.b1[j] = 0x1000
    an = _lib.Anchors()
    an.A = (1 << 24) + 1
    an.anchor = an.feat = an.offset = an.scaling = an.visible_mask = an.campos = 0x1000
    rc = lib.gs355_decode_count_static(C.byref(d), C.byref(an), 0x1000, 0x1000, None)  # rejected before any HIP call
    assert rc == _lib.GS355_ENOSPC and b"at most" in lib.gs355_last_error()
