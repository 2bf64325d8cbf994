"""CPU oracle of the Scaffold-GS / Octree-GS anchor decode.

TEST INFRASTRUCTURE ONLY.  A torch-CPU fp32 restatement of
`AnchorDecoder.forward` in eval mode (landmark/nerf_components/
model_components/fields/anchor_decoder.py:108-242; MLP shapes :79-104) for the
configuration the reference's Scaffold-GS model uses (`use_feat_bank=False`,
no level / appearance inputs; scaffold_gs/gs_model.py:126-134):

    view = anchor - camera_center ; dist = |view| ; view /= dist
    h    = [feat | view | dist]            (dist dropped for heads whose add_*_dist is False)
    opacity = tanh   (Linear(32,n)   (relu(Linear(in,32)(h))))      [A_vis, n]
    cov     =         Linear(32,7n)  (relu(Linear(in,32)(h)))       [A_vis, 7n] -> [A_vis*n, 7]
    color   = sigmoid(Linear(32,3n)  (relu(Linear(in,32)(h))))      [A_vis, 3n] -> [A_vis*n, 3]
    mask    = opacity.reshape(-1) > 0
    scaling = anchor_scaling[:, 3:6] * sigmoid(cov[:, 0:3]) ; rot = normalize(cov[:, 3:7])
    xyz     = anchor + offset * anchor_scaling[:, 0:3]

Optional branches of the reference module (same file): the feature bank
(:163-177: a softmax-weighted mix of the feature vector with its 4x and 2x
strided, tiled copies), the level input (:179-186, including the assignment
at :182 that leaves BOTH head inputs as [feat | view | level], without the
distance) and the training-mode by-products neural_opacity / mask (:239-242).

Pins (tests/test_oracle_anchor.py): the MLPs against torch.nn.Sequential
modules built exactly as the reference builds them, output count =
(opacity > 0).sum(), unit quaternions, xyz - anchor = offset * scale, colour in
(0,1), and equality of this "mask-then-compute" formulation with the
reference's "concatenate, mask, split" formulation restated with einops.
"""
import torch
import torch.nn.functional as F

HEADS = ("opacity", "cov", "color")


def mlp(h, params):
    w0, b0, w1, b1 = params
    return F.linear(F.relu(F.linear(h, w0, b0)), w1, b1)


def bank_mix(feat, weights):
    """feat'[:, j] = feat[:, 4 (j mod 8)] w0 + feat[:, 2 (j mod 16)] w1 + feat[:, j] w2  (feat [N,32], weights [N,3]):
    the reference tiles the stride-4 copy four times and the stride-2 copy twice (anchor_decoder.py:171-176)."""
    j = torch.arange(feat.shape[1])
    return (feat[:, 4 * (j % 8)] * weights[:, 0:1] + feat[:, 2 * (j % 16)] * weights[:, 1:2]
            + feat * weights[:, 2:3])


def decode(camera_center, anchor, anchor_feat, offset, scaling, visible_mask, mlps, n_offsets=10,
           add_dist=(True, True, True), keep_override=None, level=None, add_level=False, bank=None,
           dtype=torch.float32):
    """mlps: {"opacity"|"cov"|"color": (W0[32,in], b0[32], W1[k,32], b1[k])}.
    Returns xyz[G,3], color[G,3], opacity[G,1], scaling[G,3], rot[G,4] and the
    flat keep mask over (visible anchor, offset).  `keep_override` (flat bool
    over (visible anchor, offset)) replaces the mask opacity > 0: tests use it
    to obtain the values of offsets whose opacity is within rounding of zero.
    `level` [A] or [A,1] with `add_level`: every head reads [feat | view | level].
    `bank` = (W0[32,3 or 4], b0[32], W1[3,32], b1[3]) of mlp_feature_bank.
    `dtype`: torch.float64 evaluates the same statements in double precision (inputs that require grad keep their
    graph: the reference for the gradients of the training path)."""
    if visible_mask is None:
        visible_mask = torch.ones(anchor.shape[0], dtype=torch.bool)
    a = anchor[visible_mask].to(dtype)
    feat = anchor_feat[visible_mask].to(dtype)
    off = offset[visible_mask].to(dtype)
    sc = scaling[visible_mask].to(dtype)
    lvl = level.reshape(-1, 1)[visible_mask].to(dtype) if (add_level and level is not None) else None
    view = a - camera_center.to(dtype)
    dist = view.norm(dim=1, keepdim=True)
    view = view / dist
    if bank is not None:
        cat_view = torch.cat([view, lvl], dim=1) if lvl is not None else view
        feat = bank_mix(feat, torch.softmax(mlp(cat_view, bank), dim=1))
    if lvl is not None:
        with_dist = without = torch.cat([feat, view, lvl], dim=1)
    else:
        with_dist = torch.cat([feat, view, dist], dim=1)
        without = torch.cat([feat, view], dim=1)
    outs = {}
    for head, use_dist in zip(HEADS, add_dist):
        outs[head] = mlp(with_dist if use_dist else without, mlps[head])
    neural_opacity = torch.tanh(outs["opacity"]).reshape(-1, 1)
    keep = (neural_opacity > 0.0).view(-1) if keep_override is None else keep_override.view(-1).bool()
    color = torch.sigmoid(outs["color"]).reshape(-1, 3)[keep]
    cov = outs["cov"].reshape(-1, 7)[keep]
    rep = torch.arange(a.shape[0]).repeat_interleave(n_offsets)[keep]
    scaling_out = sc[rep, 3:6] * torch.sigmoid(cov[:, 0:3])
    rot = F.normalize(cov[:, 3:7])
    xyz = a[rep] + off.reshape(-1, 3)[keep] * sc[rep, 0:3]
    return dict(xyz=xyz, color=color, opacity=neural_opacity[keep], scaling=scaling_out, rot=rot, keep=keep,
                raw_opacity=neural_opacity.view(-1), neural_opacity=neural_opacity,
                mask=(neural_opacity > 0.0).view(-1))
