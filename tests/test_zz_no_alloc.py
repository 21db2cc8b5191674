"""The entry point that allocates nothing: svox_volume_render_backward_static against
svox_volume_render_backward_ws (same kernels, the workspace inside the library instead of the caller's).

Bar: gradients within 1e-4 relative of the existing entry point's (atomic summation order differs from
call to call), on two calls in a row that share the library's array, the second with fewer rays.
"""
import numpy as np
import pytest
import torch

from svox_amd import csrc as C
from svox_amd import synth
from svox_amd.csrc import _abi
from util import grad_close, on_gpu, options, rays_spec

pytestmark = pytest.mark.gpu


def test_static_workspace_backward_matches_the_workspace_entry_point(gpu, oracle_mod):
    tree = synth.shell_tree(depth=6, n_spheres=6, data_format="SH9", seed=41, sigma_range=(20.0, 200.0))
    dev = on_gpu(tree, gpu)
    ot = oracle_mod.Tree.from_n3tree(tree)
    opt = options(tree, step_size=1e-3)
    grad_static = torch.empty_like(dev.data)
    for call, (n_rays, seed) in enumerate([(20000, 7), (3000, 8)]):
        print(f"[no_alloc] call {call}: svox_volume_render_backward_static, {n_rays} rays, seed {seed}", flush=True)
        rays = synth.sphere_rays(n_rays, seed=seed)
        spec = rays_spec(rays, gpu)
        go = (torch.randn(n_rays, 3, generator=torch.Generator().manual_seed(seed + 100)) * 1e-2).to(gpu)
        reference = C.volume_render_backward(dev._spec(), spec, opt, go, workspace=True)
        grad_static.fill_(float("nan"))    # the call zero-fills its output itself
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info(gpu)[0]
        allocated_before = torch.cuda.memory_allocated(gpu)
        got = C.volume_render_backward_static(dev._spec(), spec, opt, go, grad_static)
        torch.cuda.synchronize()
        assert got is grad_static
        assert torch.cuda.memory_allocated(gpu) == allocated_before
        if call > 0:   # (the first call of a process may load the kernel's code; later ones hold what they have)
            assert torch.cuda.mem_get_info(gpu)[0] == free_before, "device memory was taken during the call"
        err, ok = grad_close(got.cpu().numpy(), reference.cpu().numpy())
        assert ok, f"call {call}: worst relative error {err:.3e} against svox_volume_render_backward_ws"
        # and against the CPU oracle, like every other gradient test
        ref_grad = oracle_mod.volume_render_backward(ot, rays.origins, rays.dirs, rays.viewdirs, opt, go.cpu())
        err, ok = grad_close(got.cpu().numpy(), ref_grad)
        assert ok, f"call {call}: worst relative error {err:.3e} against the oracle"
    # accumulate = 1 adds to what is there
    C.volume_render_backward_static(dev._spec(), spec, opt, go, grad_static, accumulate=True)
    err, ok = grad_close(grad_static.cpu().numpy(), 2.0 * reference.cpu().numpy())
    assert ok, f"accumulate: {err:.3e}"


def test_static_workspace_rejects_more_rays_than_it_serves(gpu):
    tree = synth.dense_tree(2, "RGBA", seed=0)
    dev = on_gpu(tree, gpu)
    opt = options(tree, step_size=1e-2)
    n = _abi.STATIC_RAYS_MAX + 1
    rays = synth.sphere_rays(n, seed=1)
    go = torch.zeros(n, 3, device=gpu)
    out = torch.zeros_like(dev.data)
    with pytest.raises(RuntimeError, match="exceed the 65536 rays"):
        C.volume_render_backward_static(dev._spec(), rays_spec(rays, gpu), opt, go, out)
    assert float(out.abs().max()) == 0.0   # rejected before anything ran
    # exactly the maximum is served
    rays = synth.sphere_rays(_abi.STATIC_RAYS_MAX, seed=1)
    go = torch.ones(_abi.STATIC_RAYS_MAX, 3, device=gpu)
    reference = C.volume_render_backward(dev._spec(), rays_spec(rays, gpu), opt, go)
    got = C.volume_render_backward_static(dev._spec(), rays_spec(rays, gpu), opt, go, out)
    err, ok = grad_close(got.cpu().numpy(), reference.cpu().numpy())
    assert ok, err
