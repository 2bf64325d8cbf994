"""Error metrics of a rendered frame against the oracle's frame.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.  One
definition of the numbers that the image comparisons of the tests assert and
that the benchmark publishes as its `parity` object, so that both speak of the
same quantities:

  * `fragile`: pixels on which the oracle took at least one blend decision
    within rounding distance of its threshold (alpha < 1/255, T(1-alpha) < 1e-4,
    power > 0); all other pixels are "solid";
  * per output plane (image, depth, alpha): the largest absolute error over the
    solid pixels, over all pixels, the number of pixels whose error exceeds
    1e-4, and the PSNR on the peak-normalised plane.
"""
import math

import numpy as np

IMG_TOL = 1e-4       # max-abs bar of image, alpha and depth on solid pixels
DEPTH_REL = 2.5e-5   # depth is a sum of terms up to the largest view depth: bar = max(IMG_TOL, DEPTH_REL * largest depth of the frame)
PSNR_MIN = 60.0


def psnr(a, b):
    mse = float(np.mean((np.asarray(a, np.float64) - np.asarray(b, np.float64)) ** 2))
    return float("inf") if mse == 0 else -10.0 * math.log10(mse)


def plane_errors(got, ref, want_depth=True, want_alpha=True):
    """`got`: dict with image [3,H,W] and optionally depth / alpha (any shape of H*W elements); `ref`: the oracle's
    render output (image, depth, alpha, fragile).  Returns (n_fragile, n_pixels, {plane: numbers}) where numbers =
    dict(solid=, all=, over_tol=, psnr=, bar=, peak=)."""
    frag = np.asarray(ref["fragile"])
    solid = frag == 0
    planes = [("image", np.asarray(got["image"]), ref["image"], IMG_TOL, 1.0)]
    if want_depth and got.get("depth") is not None:
        peak = max(1.0, float(np.abs(ref["depth"]).max()))
        planes.append(("depth", np.asarray(got["depth"]).reshape(ref["depth"].shape), ref["depth"],
                       max(IMG_TOL, DEPTH_REL * peak), peak))
    if want_alpha and got.get("alpha") is not None:
        planes.append(("alpha", np.asarray(got["alpha"]).reshape(ref["alpha"].shape), ref["alpha"], IMG_TOL, 1.0))
    report = {}
    for name, g, r, bar, peak in planes:
        diff = np.abs(g.astype(np.float64) - r.astype(np.float64))
        per_pixel = diff.max(axis=0) if diff.ndim == 3 else diff
        report[name] = dict(
            solid=float(per_pixel[solid].max()) if solid.any() else 0.0,
            all=float(per_pixel.max()) if per_pixel.size else 0.0,
            over_tol=int((per_pixel > IMG_TOL).sum()),
            over_bar=int((per_pixel > bar).sum()),
            psnr=psnr(g / peak, r / peak), bar=bar, peak=peak, diff=diff)
    return int((~solid).sum()), int(solid.size), report


def parity_object(got, ref, integers=None):
    """The `parity` object of the bench line: `integers` = dict of name -> bool for the bit-exact comparisons made
    by the caller (radii, keys, order, ranges)."""
    n_fragile, n_pixels, report = plane_errors(got, ref)
    out = {"checker": "oracle/gs_oracle.c over the whole frame, in this run",
           "bit_exact": dict(integers or {}),
           "pixels": n_pixels, "threshold_adjacent_pixels": n_fragile}
    for name, r in report.items():
        out[name] = {"max_abs_solid_pixels": float("%.3g" % r["solid"]), "max_abs_all_pixels": float("%.3g" % r["all"]),
                     "pixels_over_1e-4": r["over_tol"], "psnr_db": round(min(r["psnr"], 999.0), 1),
                     "solid_bar": float("%.3g" % r["bar"])}
    return out
