"""se_grad / se_grad_persp on the GPU against the oracle (reference: rt_kernel.cu:479-715, 846-897,
1111-1173): rendered colour bit-exact, gradient and Hessian diagonal within 1e-4 relative
(atomic summation order)."""
import numpy as np
import pytest
import torch

import svox_amd as svox
from svox_amd import csrc as C
from svox_amd import synth
from util import cam_spec, grad_close, on_gpu, options, rays_spec

pytestmark = pytest.mark.gpu


# how a call reaches the kernels: debug flags and whether the rays' notes are kept in a workspace
PATHS = {"generic": (1, False), "marches": (0, False), "notes": (0, True),
         "marches_large_batch_kernels": (2, False), "notes_large_batch_kernels": (2, True)}


def check(gpu, oracle_mod, tree, rays, ref, opt, exact=True, path="notes"):
    ot = oracle_mod.Tree.from_n3tree(tree)
    want = oracle_mod.se_grad(ot, rays.origins, rays.dirs, rays.viewdirs, ref, opt, n_threads=4)
    dev = on_gpu(tree, gpu)
    flags, workspace = PATHS[path]
    C.set_debug_flags(flags)
    try:
        got = C.se_grad(dev._spec(), rays_spec(rays, gpu), ref.to(gpu), opt, workspace=workspace)
    finally:
        C.set_debug_flags(0)
    got = [x.cpu().numpy() for x in got]
    if exact:
        assert np.array_equal(got[0], want[0])
    else:
        assert np.abs(got[0] - want[0]).max() <= 1e-5
    for name, g, w in (("grad", got[1], want[1]), ("hessdiag", got[2], want[2])):
        assert g.shape == tuple(tree.data.shape)
        err, ok = grad_close(g, w)
        assert ok, (name, err)
    return got, want


@pytest.mark.parametrize("path", list(PATHS))
@pytest.mark.parametrize("fmt", ["RGBA", "SH1", "SH4", "SH9", "SH16", "SH25"])
def test_se_grad_sparse_tree(gpu, oracle_mod, fmt, path):
    tree = synth.shell_tree(depth=6, n_spheres=6, data_format=fmt, seed=21, sigma_range=(20.0, 200.0))
    rays = synth.sphere_rays(3000, seed=5)
    o = rays.origins.clone()
    o[:50] += 3.0                                                  # these miss the cube
    o[50:100] = torch.rand(50, 3, generator=torch.Generator().manual_seed(2))   # these start inside
    rays = svox.Rays(o.contiguous(), rays.dirs, rays.viewdirs)
    ref = torch.rand(3000, 3, generator=torch.Generator().manual_seed(7))
    opt = options(tree, step_size=5e-4, background_brightness=0.8)
    got, want = check(gpu, oracle_mod, tree, rays, ref, opt, path=path)
    assert np.all(got[0][:50] == np.float32(0.8))
    assert np.abs(want[2]).max() > 0


def test_se_grad_equals_backward_of_the_residual(gpu):
    """Without the oracle: grad = volume_render_backward(render - color); colour = volume_render."""
    tree = synth.shell_tree(depth=7, n_spheres=8, data_format="SH16", seed=3).to(gpu)
    rays = synth.sphere_rays(20000, seed=1)
    rs = rays_spec(rays, gpu)
    ref = torch.rand(20000, 3, generator=torch.Generator().manual_seed(0)).to(gpu)
    r = svox.VolumeRenderer(tree, step_size=1e-3)
    colour, grad, hess = r.se_grad(svox.Rays(rs.origins, rs.dirs, rs.vdirs), ref)
    opt = r._get_options(False)
    plain = C.volume_render(tree._spec(), rs, opt)
    assert (colour - plain).abs().max().item() <= 1e-6
    want = C.volume_render_backward(tree._spec(), rs, opt, (colour - ref).contiguous())
    err, ok = grad_close(grad.cpu().numpy(), want.cpu().numpy())
    assert ok, err
    assert (hess >= 0).all().item() and hess.max().item() > 0


def test_se_grad_generic_options_and_double(gpu, oracle_mod):
    rays = synth.sphere_rays(1200, seed=9)
    ref = torch.rand(1200, 3, generator=torch.Generator().manual_seed(5))
    t = synth.dense_tree(2, "SH9", seed=3, sigma="lognormal", coeff_std=0.5)
    check(gpu, oracle_mod, t, rays, ref, options(t, step_size=2e-3, min_comp=1, max_comp=3))
    check(gpu, oracle_mod, t, rays, ref, options(t, step_size=2e-3, density_softplus=True, rgb_padding=0.001),
          exact=False)
    t = svox.N3Tree(N=3, data_format="SH4", init_refine=2)
    g = torch.Generator().manual_seed(6)
    t.data.data.normal_(generator=g)
    t.data.data[..., -1] = t.data.data[..., -1].abs() * 8
    check(gpu, oracle_mod, t, rays, ref, options(t, step_size=2e-3))
    t = synth.dense_tree(2, "SH4", seed=8, sigma="lognormal", dtype=torch.float64)
    r64 = svox.Rays(rays.origins.double(), rays.dirs.double(), rays.viewdirs.double())
    check(gpu, oracle_mod, t, r64, ref.double(), options(t, step_size=2e-3))


@pytest.mark.parametrize("fmt", ["RGBA", "SH9", "SH25"])
def test_se_grad_rays_whose_notes_do_not_fit(gpu, oracle_mod, fmt):
    """Through the C ABI with the smallest workspace (one chunk of 15 notes per ray and nothing to
    spare) on a dense tree: rays with more leaves than that are marked and marched, the others are
    done from their notes; together they give the oracle's result."""
    import ctypes
    from svox_amd.csrc import _abi
    tree = synth.dense_tree(3, fmt, seed=4, sigma="lognormal", coeff_std=0.5)
    n = 1500
    rays = synth.sphere_rays(n, seed=11)
    ref = torch.rand(n, 3, generator=torch.Generator().manual_seed(3))
    opt = options(tree, step_size=1e-3)
    want = oracle_mod.se_grad(oracle_mod.Tree.from_n3tree(tree), rays.origins, rays.dirs, rays.viewdirs, ref, opt,
                              n_threads=4)
    dev = on_gpu(tree, gpu)
    lib = _abi.load_library()
    spec = C._pack_tree(dev._spec())
    dev_rays = rays_spec(rays, gpu)            # owns the device tensors the packed struct points to
    rs = C._pack_rays(dev_rays, torch.float32)
    copt = opt._pack()
    nbytes = int(lib.svox_volume_render_backward_workspace_bytes(n, 15))
    ws = torch.zeros(nbytes // 8, dtype=torch.float64, device=gpu)
    colour = torch.empty(n, 3, device=gpu)
    grad = torch.empty_like(dev.data)
    hess = torch.empty_like(dev.data)
    ref_dev = ref.to(gpu)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.svox_se_grad_ws(ctypes.byref(spec), ctypes.byref(rs), ctypes.byref(copt), ref_dev.data_ptr(),
                             colour.data_ptr(), grad.data_ptr(), hess.data_ptr(), ws.data_ptr(), nbytes, stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert np.array_equal(colour.cpu().numpy(), want[0])
    for name, g, w in (("grad", grad, want[1]), ("hessdiag", hess, want[2])):
        err, ok = grad_close(g.cpu().numpy(), w)
        assert ok, (name, err)
    # the bitmap of the rays left to the marching kernel sits behind the n chunks of 384 bytes
    words = ws.view(torch.int64)[n * 384 // 8: n * 384 // 8 + (n + 63) // 64].cpu().numpy().view(np.uint64)
    undone = sum(bin(int(w)).count("1") for w in words)
    assert 0 < undone < n, undone


@pytest.mark.parametrize("workspace", [False, True])
@pytest.mark.parametrize("ndc", [False, True])
def test_se_grad_persp(gpu, oracle_mod, ndc, workspace):
    tree = synth.shell_tree(depth=6, n_spheres=5, data_format="SH9", seed=33,
                            geometry="noise" if ndc else "spheres")
    W, H, fx = 75, 53, 60.0
    if ndc:
        c2w = torch.tensor([[1.0, 0, 0, 0.1], [0, 1, 0, -0.05], [0, 0, 1, 0.3]])
        kw = dict(ndc=svox.NDCConfig(W, H, fx))
        tree.invradius.data[:] = 0.5
        tree.offset.data[:] = 0.5
    else:
        c2w = synth.orbit_poses(1, seed=4, radius=2.5)[0]
        kw = {}
    ref = torch.rand(H, W, 3, generator=torch.Generator().manual_seed(9))
    opt = options(tree, step_size=1e-3, **kw)
    want = oracle_mod.se_grad_image(oracle_mod.Tree.from_n3tree(tree), c2w, fx, fx, W, H, ref, opt, n_threads=4)
    dev = on_gpu(tree, gpu)
    r = svox.VolumeRenderer(dev, step_size=1e-3, **kw)
    cam = cam_spec(c2w.to(gpu), W, H, fx)
    got = C.se_grad_persp(dev._spec(), cam, r._get_options(False), ref.to(gpu), workspace=workspace)
    if workspace:
        again = r.se_grad_persp(c2w.to(gpu), ref.to(gpu), width=W, height=H, fx=fx)   # the renderer's default
        assert torch.equal(again[0], got[0])
    assert got[0].shape == (H, W, 3)
    assert np.array_equal(got[0].cpu().numpy(), want[0])
    for g, w in zip(got[1:], want[1:]):
        err, ok = grad_close(g.cpu().numpy(), w)
        assert ok, err


def test_se_grad_argument_checks(gpu):
    tree = synth.dense_tree(2, "SH4", seed=1).to(gpu)
    rays = synth.sphere_rays(8, seed=0)
    r = svox.VolumeRenderer(tree)
    dev_rays = svox.Rays(rays.origins.to(gpu), rays.dirs.to(gpu), rays.viewdirs.to(gpu))
    with pytest.raises(RuntimeError, match="shape"):
        r.se_grad(dev_rays, torch.zeros(7, 3, device=gpu))
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        r.se_grad(dev_rays, torch.zeros(8, 3))
    wide = svox.N3Tree(data_format="RGBA", data_dim=6, init_refine=1).to(gpu)   # 5 colour channels
    with pytest.raises(RuntimeError, match="cannot be > 4"):
        svox.VolumeRenderer(wide).se_grad(dev_rays, torch.zeros(8, 5, device=gpu))
    colour, grad, hess = r.se_grad(svox.Rays(dev_rays.origins[:0], dev_rays.dirs[:0], dev_rays.viewdirs[:0]),
                                   torch.zeros(0, 3, device=gpu))
    assert colour.shape == (0, 3) and not grad.any().item() and not hess.any().item()


def test_se_grad_ws_argument_handling(gpu):
    """svox_se_grad_ws / svox_se_grad_image_ws through the C ABI: a negative workspace size is an error;
    without a workspace, or with one too small to hold a chunk per ray, the call is the plain one."""
    import ctypes
    from svox_amd.csrc import _abi
    tree = synth.shell_tree(depth=5, n_spheres=4, data_format="SH4", seed=2, sigma_range=(2.0, 20.0)).to(gpu)
    n = 700
    rays = synth.sphere_rays(n, seed=1)
    dev_rays = rays_spec(rays, gpu)
    opt = options(tree, step_size=1e-3)
    ref = torch.rand(n, 3, generator=torch.Generator().manual_seed(3)).to(gpu)
    want = C.se_grad(tree._spec(), dev_rays, ref, opt, workspace=False)
    lib = _abi.load_library()
    spec = C._pack_tree(tree._spec())
    rs = C._pack_rays(dev_rays, torch.float32)
    copt = opt._pack()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    colour = torch.empty(n, 3, device=gpu)
    grad = torch.empty_like(tree.data)
    hess = torch.empty_like(tree.data)
    small = torch.empty(n * 384 // 8, dtype=torch.float64, device=gpu)     # no room for bitmap and bookkeeping

    def call(ws, nbytes):
        return lib.svox_se_grad_ws(ctypes.byref(spec), ctypes.byref(rs), ctypes.byref(copt), ref.data_ptr(),
                                   colour.data_ptr(), grad.data_ptr(), hess.data_ptr(), ws, nbytes, stream)

    assert call(None, -1) < 0 and b"negative" in lib.svox_last_error()
    for ws, nbytes in ((None, 0), (small.data_ptr(), small.numel() * 8)):
        colour.fill_(-1.0)
        assert call(ws, nbytes) == 0
        torch.cuda.synchronize()
        assert torch.equal(colour, want[0])
        for g, w in ((grad, want[1]), (hess, want[2])):
            err, ok = grad_close(g.cpu().numpy(), w.cpu().numpy())
            assert ok, err
    cam = C._pack_camera(cam_spec(synth.orbit_poses(1, seed=4, radius=2.5)[0].to(gpu), 40, 30, 35.0), torch.float32)
    img_ref = torch.rand(30, 40, 3, device=gpu)
    img = torch.empty(30, 40, 3, device=gpu)
    rc = lib.svox_se_grad_image_ws(ctypes.byref(spec), ctypes.byref(cam), ctypes.byref(copt), img_ref.data_ptr(),
                                   img.data_ptr(), grad.data_ptr(), hess.data_ptr(), None, -8, stream)
    assert rc < 0 and b"negative" in lib.svox_last_error()
