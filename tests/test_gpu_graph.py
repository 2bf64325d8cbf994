"""The C entry points enqueue kernels on the caller's stream and nothing else (no allocation, no memset, no
synchronisation), so a frame can be captured into a HIP graph and replayed with new camera matrices written into the
same device tensors.  Replays are interleaved with eager work and synchronisations and every replay is compared
with an eager render of the same camera."""
import math

import numpy as np
import pytest
import torch

from landmarksystem_amd import GaussianRasterizationSettings, _lib, pipeline, scenes

pytestmark = pytest.mark.gpu


def _settings(scene, cam, view, proj, campos, bg):
    return GaussianRasterizationSettings(
        image_height=int(cam.height), image_width=int(cam.width), tanfovx=math.tan(cam.FovX * 0.5),
        tanfovy=math.tan(cam.FovY * 0.5), bg=bg,
        scale_modifier=1.0, viewmatrix=view, projmatrix=proj, sh_degree=scene.sh_degree, campos=campos,
        prefiltered=False, debug=False)


@pytest.mark.parametrize("modifier", [0, _lib.STAGE_TILE_SCATTER_ONE_LEVEL, _lib.STAGE_TILE_SCATTER_TWO_LEVEL])
def test_captured_frame_replays_with_new_cameras(gpu_device, modifier):
    dev = gpu_device
    scene = scenes.config4(P=200_000, width=640, height=360, n_poses=5)
    d = scene.to(dev)
    cams = d.cameras
    view = cams[0].world_view_transform.clone().contiguous()
    proj = cams[0].full_proj_transform.clone().contiguous()
    campos = cams[0].camera_center.clone().contiguous()
    bg = d.bg
    inp = pipeline.FrameInputs(_settings(scene, cams[0], view, proj, campos, bg), d.means3D, opacities=d.opacities,
                               shs=d.shs, scales=d.scales, rotations=d.rotations)
    assert inp.viewmatrix.data_ptr() == view.data_ptr()  # the frame reads these tensors in place
    out = pipeline.FrameOutputs(inp)
    ws = pipeline.Workspace(dev)
    n_cap = 8 * scene.P
    mask = _lib.PIPELINE_FAST | modifier

    side = torch.cuda.Stream(dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):  # first call outside the capture: sizes the workspace, sets the kernels' LDS limits
        lay = pipeline.run_stages(inp, out, ws, n_cap, mask)
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        pipeline.run_stages(inp, out, ws, n_cap, mask)

    for k in (1, 3, 0, 4, 2, 2):
        cam = cams[k]
        view.copy_(cam.world_view_transform)
        proj.copy_(cam.full_proj_transform)
        campos.copy_(cam.camera_center)
        graph.replay()
        torch.cuda.synchronize()
        got = {n: getattr(out, n).clone() for n in ("image", "depth", "alpha", "radii")}
        # eager work between the replays: the same camera rendered through the ordinary path, its own workspace
        ref_inp = pipeline.FrameInputs(_settings(scene, cam, cam.world_view_transform, cam.full_proj_transform,
                                                 cam.camera_center, bg), d.means3D, opacities=d.opacities,
                                       shs=d.shs, scales=d.scales, rotations=d.rotations)
        ref = pipeline.render(ref_inp, ws=pipeline.Workspace(dev))
        torch.cuda.synchronize()
        header = ws.view(lay, "header", inp.P, 0, inp.tiles).cpu()
        assert int(header[0]) == ref.num_keys > 0 and ((int(header[1]) >> 32) & 0xFFFFFFFF) == 0, "pose %d" % k
        for n in got:
            np.testing.assert_array_equal(got[n].cpu().numpy(), getattr(ref, n).cpu().numpy(), err_msg="pose %d %s" % (k, n))
