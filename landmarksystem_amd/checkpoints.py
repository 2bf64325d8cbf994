"""Checkpoint I/O for the three Gaussian-splatting encodings: `point_cloud.ply`
(per-Gaussian / per-anchor parameters) plus `state_dict.th` (decoder MLPs).

The reference reads and writes these files through the third-party `plyfile`
package; this module carries its own reader / writer for the subset of the
PLY format those files use (one `vertex` element of scalar properties,
ascii or binary of either endianness), so trained scenes can flow into the
renderer without that dependency.

  vanilla 3DGS   landmark/nerf_components/model_components/fields/encodings/
                 gaussian_encoding.py:154-271 (read), :340-404 (write + column order)
  Scaffold-GS    .../encodings/scaffoldgs_encoding.py:163-235 (read), :283-325 (write)
  Octree-GS      .../encodings/octreegs_encoding.py:296-372 (read), :413-466 (write)
  directory      landmark/nerf_components/model/base_model.py:249-342
                 (`point_cloud.ply` + `state_dict.th`, merged on load; duplicates are an error)

Column conventions kept from the reference: `f_rest_*` and `cache_f_*` are
stored channel-major (all coefficients of red, then green, then blue) and
come back as `[P, coeffs, 3]`; `f_offset_*` is stored axis-major (all x, then
y, then z) and comes back as `[A, n_offsets, 3]`; Octree-GS keeps
`voxel_size` and `standard_dist` in rows 0 and 1 of an `info` column.
"""
import os
import re
from typing import Dict, List, Mapping, Optional, Sequence, Tuple

import numpy as np
import torch

_PLY_SCALARS = {
    "char": "i1", "int8": "i1", "uchar": "u1", "uint8": "u1",
    "short": "i2", "int16": "i2", "ushort": "u2", "uint16": "u2",
    "int": "i4", "int32": "i4", "uint": "u4", "uint32": "u4",
    "float": "f4", "float32": "f4", "double": "f8", "float64": "f8",
}
_MAX_HEADER_BYTES = 1 << 20


class PlyError(ValueError):
    pass


class PlyVertices:
    """First element of a PLY file, column-addressable (the reference only ever reads `elements[0]`)."""

    def __init__(self, names: List[str], table: np.ndarray):
        self.names = names
        self._table = table  # structured array [N] or plain float32 matrix [N, K]

    def __len__(self) -> int:
        return self._table.shape[0]

    def __contains__(self, name: str) -> bool:
        return name in self.names

    def column(self, name: str) -> np.ndarray:
        if name not in self.names:
            raise KeyError(name)
        if self._table.dtype.names is None:
            return self._table[:, self.names.index(name)]
        return self._table[name]

    def columns(self, names: Sequence[str]) -> np.ndarray:
        """float32 matrix [N, len(names)] in the given column order."""
        if self._table.dtype.names is None:
            idx = [self.names.index(n) for n in names]
            if idx and idx == list(range(idx[0], idx[0] + len(idx))):
                return np.ascontiguousarray(self._table[:, idx[0]:idx[0] + len(idx)])
            return np.ascontiguousarray(self._table[:, idx])
        out = np.empty((len(self), len(names)), dtype=np.float32)
        for k, n in enumerate(names):
            out[:, k] = self._table[n]
        return out

    def numbered(self, prefix: str) -> List[str]:
        """Property names starting with `prefix`, ordered by their trailing integer (gaussian_encoding.py:192-193)."""
        found = [n for n in self.names if n.startswith(prefix)]
        return sorted(found, key=lambda n: int(n.split("_")[-1]))


def _parse_header(fh) -> Tuple[str, List[Tuple[str, int, List[Tuple[str, str]]]], int]:
    raw = fh.read(_MAX_HEADER_BYTES)
    m = re.search(rb"end_header\r?\n", raw)
    if not raw.startswith(b"ply") or m is None:
        raise PlyError("not a PLY file (missing 'ply' magic or 'end_header')")
    lines = raw[:m.start()].decode("ascii", errors="replace").splitlines()
    fmt = None
    elements: List[Tuple[str, int, List[Tuple[str, str]]]] = []
    for line in lines[1:]:
        tok = line.split()
        if not tok or tok[0] in ("comment", "obj_info"):
            continue
        if tok[0] == "format":
            if len(tok) != 3 or tok[2] != "1.0":
                raise PlyError("unsupported PLY format line: %r" % line)
            fmt = tok[1]
        elif tok[0] == "element":
            elements.append((tok[1], int(tok[2]), []))
        elif tok[0] == "property":
            if not elements:
                raise PlyError("property before any element")
            if tok[1] == "list":
                elements[-1][2].append((tok[-1], "list"))
            else:
                if tok[1] not in _PLY_SCALARS:
                    raise PlyError("unknown PLY scalar type %r" % tok[1])
                elements[-1][2].append((tok[2], _PLY_SCALARS[tok[1]]))
        else:
            raise PlyError("unexpected header line: %r" % line)
    if fmt not in ("ascii", "binary_little_endian", "binary_big_endian"):
        raise PlyError("unsupported PLY format %r" % fmt)
    if not elements:
        raise PlyError("PLY file declares no element")
    return fmt, elements, m.end()


def read_ply(path) -> PlyVertices:
    """Read the first element of a PLY file.  An all-float32 little-endian table (what every writer of these
    checkpoints produces) is returned as one [N, K] matrix without a per-column copy."""
    with open(path, "rb") as fh:
        fmt, elements, data_start = _parse_header(fh)
        _, count, props = elements[0]
        if any(t == "list" for _, t in props):
            raise PlyError("list properties in the first element are not supported")
        names = [n for n, _ in props]
        if len(set(names)) != len(names):
            raise PlyError("duplicate property names in the first element")
        fh.seek(data_start)
        if fmt == "ascii":
            flat = np.array(fh.read().split()[:count * len(props)], dtype=np.float64)
            if flat.size != count * len(props):
                raise PlyError("ascii PLY body is shorter than the header declares")
            mat = flat.reshape(count, len(props))
            table = np.empty(count, dtype=[(n, "<" + t) for n, t in props])
            for k, (n, _) in enumerate(props):
                table[n] = mat[:, k]
            return PlyVertices(names, table)
        order = "<" if fmt == "binary_little_endian" else ">"
        dtype = np.dtype([(n, order + t) for n, t in props])
        need = count * dtype.itemsize
        if order == "<" and all(t == "f4" for _, t in props):
            mat = np.fromfile(fh, dtype="<f4", count=count * len(props))
            if mat.size != count * len(props):
                raise PlyError("binary PLY body is shorter than the header declares (%d bytes needed)" % need)
            return PlyVertices(names, mat.reshape(count, len(props)))
        table = np.fromfile(fh, dtype=dtype, count=count)
        if table.shape[0] != count:
            raise PlyError("binary PLY body is shorter than the header declares (%d bytes needed)" % need)
        return PlyVertices(names, table)


def write_ply(path, names: Sequence[str], columns: np.ndarray) -> None:
    """Write one `vertex` element of float properties, binary little-endian: the file `plyfile` produces for
    the reference's all-"f4" structured arrays (gaussian_encoding.py:373-382)."""
    columns = np.ascontiguousarray(columns, dtype="<f4")
    if columns.ndim != 2 or columns.shape[1] != len(names):
        raise ValueError("columns must be [N, %d], got %r" % (len(names), columns.shape))
    header = ["ply", "format binary_little_endian 1.0", "element vertex %d" % columns.shape[0]]
    header += ["property float %s" % n for n in names]
    header.append("end_header")
    with open(path, "wb") as fh:
        fh.write(("\n".join(header) + "\n").encode("ascii"))
        columns.tofile(fh)


def _t(a: np.ndarray, device, dtype=torch.float) -> torch.Tensor:
    return torch.as_tensor(np.ascontiguousarray(a)).to(device=device, dtype=dtype)


def _channel_major(v: PlyVertices, cols: List[str], device) -> torch.Tensor:
    # stored [N, 3*k] as (channel, k); the models hold [N, k, 3]
    m = v.columns(cols)
    return _t(m, device).reshape(m.shape[0], 3, -1).transpose(1, 2).contiguous()


def gaussian_state_dict(path, max_sh_degree: int = 3, map_location="cpu", prefix: str = "") -> Dict[str, torch.Tensor]:
    """Vanilla 3DGS parameters from a PLY file (gaussian_encoding.py:154-271): either the raw schema
    (`opacity`, `f_dc_*`, `f_rest_*`, `scale_*`, `rot_*`) or the activation-cache schema (`cache_*`)."""
    v = read_ply(path)
    xyz = _t(v.columns(["x", "y", "z"]), map_location)
    n_coeff = (max_sh_degree + 1) ** 2
    if "opacity" in v:
        rest = v.numbered("f_rest_")
        if len(rest) != 3 * n_coeff - 3:
            raise PlyError("expected %d f_rest_* properties for SH degree %d, found %d"
                           % (3 * n_coeff - 3, max_sh_degree, len(rest)))
        feats_rest = (_channel_major(v, rest, map_location) if rest
                      else torch.zeros(len(v), 0, 3, device=map_location))
        return {
            prefix + "_xyz": xyz,
            prefix + "_features_dc": _channel_major(v, ["f_dc_0", "f_dc_1", "f_dc_2"], map_location),
            prefix + "_features_rest": feats_rest,
            prefix + "_opacity": _t(v.columns(["opacity"]), map_location),
            prefix + "_scaling": _t(v.columns(v.numbered("scale_")), map_location),
            prefix + "_rotation": _t(v.columns(v.numbered("rot")), map_location),
        }
    if "cache_opacity" in v:
        feats = v.numbered("cache_f_")
        if len(feats) != 3 * n_coeff:
            raise PlyError("expected %d cache_f_* properties for SH degree %d, found %d"
                           % (3 * n_coeff, max_sh_degree, len(feats)))
        return {
            prefix + "_xyz": xyz,
            prefix + "_cache_features": _channel_major(v, feats, map_location),
            prefix + "_cache_opacity": _t(v.columns(["cache_opacity"]), map_location),
            prefix + "_cache_scaling": _t(v.columns(v.numbered("cache_scale_")), map_location),
            prefix + "_cache_rotation": _t(v.columns(v.numbered("cache_rot_")), map_location),
        }
    raise NotImplementedError("unsupport keys %s" % (v.names,))


def _anchor_columns(v: PlyVertices, map_location, prefix: str) -> Dict[str, torch.Tensor]:
    return {
        prefix + "_anchor_feat": _t(v.columns(v.numbered("f_anchor_feat")), map_location),
        prefix + "_offset": _channel_major(v, v.numbered("f_offset"), map_location),
        prefix + "_anchor": _t(v.columns(["x", "y", "z"]), map_location),
        prefix + "_opacity": _t(v.columns(["opacity"]), map_location),
        prefix + "_scaling": _t(v.columns(v.numbered("scale_")), map_location),
        prefix + "_rotation": _t(v.columns(v.numbered("rot")), map_location),
    }


def scaffold_state_dict(path, map_location="cpu", prefix: str = "") -> Dict[str, torch.Tensor]:
    """Scaffold-GS anchors from a PLY file (scaffoldgs_encoding.py:163-235)."""
    return _anchor_columns(read_ply(path), map_location, prefix)


def octree_state_dict(path, map_location="cpu", prefix: str = "") -> Tuple[Dict[str, torch.Tensor], float, float]:
    """Octree-GS anchors from a PLY file (octreegs_encoding.py:296-372).  Returns the state dict and the two
    scalars the writer keeps in the `info` column: `(state, voxel_size, standard_dist)`."""
    v = read_ply(path)
    if len(v) < 2:
        raise PlyError("an Octree-GS PLY needs at least two rows (voxel_size and standard_dist live in info[0:2])")
    state = _anchor_columns(v, map_location, prefix)
    state[prefix + "_level"] = _t(v.column("level").astype(np.int64)[:, None], map_location, torch.int)
    state[prefix + "_extra_level"] = _t(v.columns(["extra_level"])[:, 0], map_location)
    info = v.column("info")
    return state, float(np.float32(info[0])), float(np.float32(info[1]))


def load_mlp_state(dir_path, map_location="cpu") -> Dict[str, torch.Tensor]:
    """`state_dict.th` beside the PLY (base_model.py:335-337); empty when the file is absent, as for vanilla 3DGS.
    Loaded with `weights_only=True`: nothing in the file is executed."""
    path = os.path.join(dir_path, "state_dict.th")
    if not os.path.exists(path):
        return {}
    return dict(torch.load(path, map_location=map_location, weights_only=True))


def merged_state_dict(ply_path, kind: str, map_location="cpu", prefix: str = "gaussian_encoding.",
                      max_sh_degree: int = 3) -> Dict[str, torch.Tensor]:
    """What the reference's `BaseGaussian.get_state_dict_from_ckpt` returns (base_model.py:308-342): the PLY
    columns under `prefix` merged with `state_dict.th` from the same directory."""
    if kind == "gaussian":
        state = gaussian_state_dict(ply_path, max_sh_degree, map_location, prefix)
    elif kind == "scaffold":
        state = scaffold_state_dict(ply_path, map_location, prefix)
    elif kind == "octree":
        state, _, _ = octree_state_dict(ply_path, map_location, prefix)  # the two scalars are not state-dict entries
    else:
        raise ValueError("kind must be 'gaussian', 'scaffold' or 'octree', got %r" % (kind,))
    extra = load_mlp_state(os.path.dirname(os.path.abspath(ply_path)), map_location)
    duplicate = set(state) & set(extra)
    if duplicate:
        raise ValueError("Duplicate keys found: %s" % (duplicate,))
    state.update(extra)
    return state


def _ply_in(path) -> str:
    return os.path.join(path, "point_cloud.ply") if os.path.isdir(path) else str(path)


def _decoder_state(state: Mapping[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    pre = "anchor_decoder."
    return {k[len(pre):]: v for k, v in state.items() if k.startswith(pre)}


def _decoder_kwargs(dec: Mapping[str, torch.Tensor], n_offsets: int, feat_dim: int, add_level: bool = False) -> Dict[str, bool]:
    # the first layer's width tells whether the camera distance is appended: feat + view(3) [+ dist(1)] [+ level(1)];
    # a feature bank shows as its own MLP, whose input width tells whether it takes the level
    out = {}
    bank = dec.get("mlp_feature_bank.0.weight")
    if bank is not None:
        out["use_feat_bank"] = True
        add_level = add_level or bank.shape[1] == 4
    if add_level:
        out["add_level"] = True
    for head in ("opacity", "cov", "color"):
        w = dec.get("mlp_%s.0.weight" % head)
        if w is not None:
            out["add_%s_dist" % head] = bool(w.shape[1] == feat_dim + 4 + (1 if add_level else 0))
    return out


def _reorder(state: Dict[str, torch.Tensor], positions: str) -> None:
    """Store the per-Gaussian / per-anchor tensors along a Morton curve of their positions (see
    `models.morton_order`): same scene, memory-coherent frames.  Indices of by-products then refer to this order."""
    from .models import morton_order
    order = morton_order(state[positions])
    n = order.shape[0]
    for k, v in state.items():
        if torch.is_tensor(v) and v.dim() >= 1 and v.shape[0] == n:
            state[k] = v[order].contiguous()


def load_gaussian_model(path, sh_degree: int = 3, device="cuda", spatial_order: bool = False, **kw):
    """`GaussianModel` from a checkpoint directory or a PLY file.  `spatial_order` stores the Gaussians along a
    Morton curve instead of in file order."""
    from .models import GaussianModel
    s = gaussian_state_dict(_ply_in(path), sh_degree, device)
    if spatial_order:
        _reorder(s, "_xyz")
    if "_cache_opacity" in s:
        return GaussianModel.from_cache(s["_xyz"], s["_cache_features"], s["_cache_scaling"], s["_cache_rotation"],
                                        s["_cache_opacity"], sh_degree=sh_degree, **kw)
    return GaussianModel(s["_xyz"], s["_features_dc"], s["_features_rest"], s["_scaling"], s["_rotation"],
                         s["_opacity"], sh_degree=sh_degree, **kw)


def load_scaffold_gs(path, device="cuda", spatial_order: bool = False, **kw):
    """`ScaffoldGS` from a checkpoint directory (`point_cloud.ply` + `state_dict.th`)."""
    from .models import ScaffoldGS
    ply = _ply_in(path)
    s = scaffold_state_dict(ply, device)
    if spatial_order:
        _reorder(s, "_anchor")
    dec = _decoder_state(load_mlp_state(os.path.dirname(os.path.abspath(ply)), device))
    n_offsets, feat_dim = s["_offset"].shape[1], s["_anchor_feat"].shape[1]
    kw = {**_decoder_kwargs(dec, n_offsets, feat_dim), **kw}
    m = ScaffoldGS(s["_anchor"], s["_anchor_feat"], s["_offset"], s["_scaling"], s["_rotation"],
                   opacity=s["_opacity"], n_offsets=n_offsets, feat_dim=feat_dim, **kw)
    if dec:
        m.anchor_decoder.load_state_dict(dec)
    return m.to(device)


def load_octree_gs(path, device="cuda", spatial_order: bool = False, **kw):
    """`OctreeGS` from a checkpoint directory (`point_cloud.ply` + `state_dict.th`)."""
    from .models import OctreeGS
    ply = _ply_in(path)
    s, voxel_size, standard_dist = octree_state_dict(ply, device)
    if spatial_order:
        _reorder(s, "_anchor")
    dec = _decoder_state(load_mlp_state(os.path.dirname(os.path.abspath(ply)), device))
    n_offsets, feat_dim = s["_offset"].shape[1], s["_anchor_feat"].shape[1]
    kw = {**_decoder_kwargs(dec, n_offsets, feat_dim, bool(kw.get("add_level", False))), **kw}
    m = OctreeGS(s["_anchor"], s["_anchor_feat"], s["_offset"], s["_scaling"], s["_rotation"], s["_level"],
                 voxel_size, standard_dist, extra_level=s["_extra_level"], opacity=s["_opacity"],
                 n_offsets=n_offsets, feat_dim=feat_dim, **kw)
    if dec:
        m.anchor_decoder.load_state_dict(dec)
    return m.to(device)


def _np(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def _flat_channel_major(t: torch.Tensor) -> np.ndarray:
    return _np(t.detach().transpose(1, 2).flatten(start_dim=1).contiguous())


def _numbered(prefix: str, n: int) -> List[str]:
    return ["%s%d" % (prefix, i) for i in range(n)]


def save_model(model, dir_path, rank: Optional[int] = None) -> None:
    """Write `point_cloud.ply` (+ `state_dict.th` for the anchor models) in the reference's layout and column
    order (base_model.py:249-306; gaussian_encoding.py:340-404; scaffoldgs_encoding.py:283-325;
    octreegs_encoding.py:413-466)."""
    from .models import GaussianModel, OctreeGS, ScaffoldGS
    os.makedirs(dir_path, exist_ok=True)
    suffix = "" if rank is None else "-sub%d" % rank
    ply = os.path.join(dir_path, "point_cloud%s.ply" % suffix)
    if isinstance(model, GaussianModel):
        xyz = _np(model._xyz)
        if model._xyz.shape[0] and model._opacity.shape[0] == 0:  # built from an activation cache
            c = model._cache
            names = (["x", "y", "z", "nx", "ny", "nz"] + _numbered("cache_f_", c["features"].shape[1] * 3)
                     + ["cache_opacity"] + _numbered("cache_scale_", c["scaling"].shape[1])
                     + _numbered("cache_rot_", c["rotation"].shape[1]))
            cols = [xyz, np.zeros_like(xyz), _flat_channel_major(c["features"]), _np(c["opacity"]),
                    _np(c["scaling"]), _np(c["rotation"])]
        else:
            names = (["x", "y", "z", "nx", "ny", "nz"] + _numbered("f_dc_", 3)
                     + _numbered("f_rest_", model._features_rest.shape[1] * 3) + ["opacity"]
                     + _numbered("scale_", model._scaling.shape[1]) + _numbered("rot_", model._rotation.shape[1]))
            cols = [xyz, np.zeros_like(xyz), _flat_channel_major(model._features_dc),
                    _flat_channel_major(model._features_rest), _np(model._opacity), _np(model._scaling),
                    _np(model._rotation)]
        write_ply(ply, names, np.concatenate(cols, axis=1))
        return
    if not isinstance(model, ScaffoldGS):
        raise TypeError("save_model expects a GaussianModel, ScaffoldGS or OctreeGS, got %s" % type(model).__name__)
    anchor = _np(model._anchor)
    tail_names = (_numbered("f_offset_", model._offset.shape[1] * 3)
                  + _numbered("f_anchor_feat_", model._anchor_feat.shape[1]) + ["opacity"]
                  + _numbered("scale_", model._scaling.shape[1]) + _numbered("rot_", model._rotation.shape[1]))
    tail = [_flat_channel_major(model._offset), _np(model._anchor_feat), _np(model._opacity), _np(model._scaling),
            _np(model._rotation)]
    if isinstance(model, OctreeGS):
        info = np.zeros((anchor.shape[0], 1), dtype=np.float32)
        info[0, 0], info[1, 0] = model.voxel_size, model.standard_dist
        names = ["x", "y", "z", "level", "extra_level", "info"] + tail_names
        cols = [anchor, _np(model._level), _np(model._extra_level)[:, None], info] + tail
    else:
        names = ["x", "y", "z", "nx", "ny", "nz"] + tail_names
        cols = [anchor, np.zeros_like(anchor)] + tail
    write_ply(ply, names, np.concatenate(cols, axis=1))
    state = {"anchor_decoder." + k: v.detach().cpu() for k, v in model.anchor_decoder.state_dict().items()}
    torch.save(state, os.path.join(dir_path, "state_dict%s.th" % suffix))
