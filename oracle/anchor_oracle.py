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


def decode(camera_center, anchor, anchor_feat, offset, scaling, visible_mask, mlps, n_offsets=10,
           add_dist=(True, True, True), keep_override=None):
    """mlps: {"opacity"|"cov"|"color": (W0[32,in], b0[32], W1[k,32], b1[k])}.
    Returns xyz[G,3], color[G,3], opacity[G,1], scaling[G,3], rot[G,4] and the
    flat keep mask over (visible anchor, offset).  `keep_override` (flat bool
    over (visible anchor, offset)) replaces the mask opacity > 0: tests use it
    to obtain the values of offsets whose opacity is within rounding of zero."""
    if visible_mask is None:
        visible_mask = torch.ones(anchor.shape[0], dtype=torch.bool)
    a = anchor[visible_mask].float()
    feat = anchor_feat[visible_mask].float()
    off = offset[visible_mask].float()
    sc = scaling[visible_mask].float()
    view = a - camera_center.float()
    dist = view.norm(dim=1, keepdim=True)
    view = view / dist
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
                raw_opacity=neural_opacity.view(-1))
