"""grid_weight_render on the GPU against the oracle (reference: rt_kernel.cu:898-1003, 1174-1203).
Maxima and visit counts do not depend on the order of the atomics: both outputs compare equal."""
import numpy as np
import pytest
import torch

import svox_amd as svox
from svox_amd import csrc as C
from svox_amd import synth
from util import cam_spec, options

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("reso", [32, 37])
def test_grid_weight_render_matches_the_oracle(gpu, oracle_mod, dtype, reso):
    g = torch.Generator().manual_seed(reso)
    data = (torch.randn(reso, reso, reso, generator=g, dtype=dtype) * 6).clamp_min(0)
    offset = torch.tensor([0.45, 0.5, 0.55], dtype=dtype)
    scaling = torch.tensor([0.8, 0.9, 1.0], dtype=dtype)
    c2w = synth.orbit_poses(1, seed=2, radius=2.2)[0]
    W, H, fx = 90, 61, 70.0
    tree = svox.N3Tree(data_format="RGBA")
    opt = options(tree, step_size=1e-3, sigma_thresh=1.0)
    want_w, want_h = oracle_mod.grid_weight_render(data, c2w, fx, fx, W, H, opt, offset, scaling)
    assert want_h.sum() > 10000
    cam = cam_spec(c2w, W, H, fx, device=gpu, dtype=dtype)
    got_w, got_h = C.grid_weight_render(data.to(gpu), cam, opt, offset.to(gpu), scaling.to(gpu))
    assert np.array_equal(got_h.cpu().numpy(), want_h)
    assert np.array_equal(got_w.cpu().numpy(), want_w)


def test_grid_weight_render_checks_and_empty_image(gpu):
    data = torch.rand(8, 8, 8, device=gpu)
    one, zero = torch.ones(3, device=gpu), torch.zeros(3, device=gpu)
    opt = options(svox.N3Tree(data_format="RGBA"))
    c2w = synth.orbit_poses(1, seed=0, radius=2.0)[0]
    w, h = C.grid_weight_render(data, cam_spec(c2w, 0, 0, 10.0, device=gpu), opt, zero, one)
    assert not w.any().item() and not h.any().item()
    with pytest.raises(RuntimeError, match="cubic"):
        C.grid_weight_render(torch.rand(8, 8, 4, device=gpu), cam_spec(c2w, 4, 4, 10.0, device=gpu), opt, zero, one)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        C.grid_weight_render(data.cpu(), cam_spec(c2w, 4, 4, 10.0, device=gpu), opt, zero, one)
    with pytest.raises(RuntimeError, match="3 elements"):
        C.grid_weight_render(data, cam_spec(c2w, 4, 4, 10.0, device=gpu), opt, zero[:2].contiguous(), one)
