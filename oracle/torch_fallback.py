"""Vectorised PyTorch restatement of the reference's CPU fallback.  TEST INFRASTRUCTURE ONLY.

The reference runs these routines when its CUDA extension is absent: the level-by-level masked
point query (svox/svox.py:224-268), the corner walk (svox/svox.py:994-1012) and the renderer that
advances all live rays one leaf at a time with a full tree query per step
(svox/renderer.py:205-282).  They are what "the reference's CPU path" means when a CPU baseline
is timed, and -- being differentiable through torch.autograd -- an independent derivation of the
gradient the backward kernels must produce.

Differences from the reference's fallback, on purpose:
  * the last line of its renderer adds a (B,) tensor to a (B, 3) tensor and only works for B = 1
    (svox/renderer.py:281); here the background term is broadcast per ray;
  * rays that miss the unit cube return the background, as the kernels do (the fallback has no miss
    test);
  * the caller's tensors are never modified in place.
It keeps the fallback's semantics otherwise: no sigma / stop thresholds, relu on sigma, RGBA and
SH only, direction normalised in world space.
"""
import torch

C0 = 0.28209479177387814
C1 = 0.4886025119029199
C2 = [1.0925484305920792, -1.0925484305920792, 0.31539156525252005, -1.0925484305920792, 0.5462742152960396]
C3 = [-0.5900435899266435, 2.890611442640554, -0.4570457994644658, 0.3731763325901154,
      -0.4570457994644658, 1.445305721320277, -0.5900435899266435]
C4 = [2.5033429417967046, -1.7701307697799304, 0.9461746957575601, -0.6690465435572892,
      0.10578554691520431, -0.6690465435572892, 0.47308734787878004, -1.7701307697799304,
      0.6258357354491761]


def eval_sh_bases(basis_dim, dirs):
    """(..., basis_dim) real SH basis in the reference's convention (svox/sh.py:113-161)."""
    out = torch.empty((*dirs.shape[:-1], basis_dim), dtype=dirs.dtype, device=dirs.device)
    out[..., 0] = C0
    if basis_dim > 1:
        x, y, z = dirs.unbind(-1)
        out[..., 1] = -C1 * y
        out[..., 2] = C1 * z
        out[..., 3] = -C1 * x
    if basis_dim > 4:
        xx, yy, zz = x * x, y * y, z * z
        xy, yz, xz = x * y, y * z, x * z
        out[..., 4] = C2[0] * xy
        out[..., 5] = C2[1] * yz
        out[..., 6] = C2[2] * (2.0 * zz - xx - yy)
        out[..., 7] = C2[3] * xz
        out[..., 8] = C2[4] * (xx - yy)
    if basis_dim > 9:
        out[..., 9] = C3[0] * y * (3 * xx - yy)
        out[..., 10] = C3[1] * xy * z
        out[..., 11] = C3[2] * y * (4 * zz - xx - yy)
        out[..., 12] = C3[3] * z * (2 * zz - 3 * xx - 3 * yy)
        out[..., 13] = C3[4] * x * (4 * zz - xx - yy)
        out[..., 14] = C3[5] * z * (xx - yy)
        out[..., 15] = C3[6] * x * (xx - 3 * yy)
    if basis_dim > 16:
        out[..., 16] = C4[0] * xy * (xx - yy)
        out[..., 17] = C4[1] * yz * (3 * xx - yy)
        out[..., 18] = C4[2] * xy * (7 * zz - 1)
        out[..., 19] = C4[3] * yz * (7 * zz - 3)
        out[..., 20] = C4[4] * (zz * (35 * zz - 30) + 3)
        out[..., 21] = C4[5] * xz * (7 * zz - 3)
        out[..., 22] = C4[6] * (xx - yy) * (7 * zz - 1)
        out[..., 23] = C4[7] * xz * (xx - 3 * yy)
        out[..., 24] = C4[8] * (xx * (xx - 3 * yy) - yy * (3 * xx - yy))
    return out


def query(data, child, points_tree, N):
    """Leaf of each tree-space point: (values (Q, K), node (Q,), cell (Q, 3), levels (Q,)).
    Masked descent, one level per iteration, as in svox/svox.py:238-262."""
    Q = points_tree.shape[0]
    pos = points_tree.clamp(0.0, 1.0 - 1e-10).clone()
    node = torch.zeros(Q, dtype=torch.long)
    cell = torch.zeros(Q, 3, dtype=torch.long)
    levels = torch.zeros(Q, dtype=torch.long)
    live = torch.arange(Q)
    cur = pos
    while live.numel():
        cur = cur * N
        fl = torch.floor(cur).clamp_max(N - 1)
        cur = cur - fl
        idx = fl.long()
        delta = child[node[live], idx[:, 0], idx[:, 1], idx[:, 2]].long()
        levels[live] += 1
        done = delta == 0
        cell[live[done]] = idx[done]
        pos[live[done]] = cur[done]
        node[live] += delta
        live = live[~done]
        cur = cur[~done]
    values = data[node, cell[:, 0], cell[:, 1], cell[:, 2]]
    return values, node, cell, levels, pos


def corners(parent_depth, node, cell, N, dtype):
    """Lower corner of each leaf by walking parent links (svox/svox.py:994-1012)."""
    out = torch.zeros(node.shape[0], 3, dtype=dtype)
    cur_node = node.clone()
    cur_cell = cell.clone()
    mask = torch.ones(node.shape[0], dtype=torch.bool)
    while True:
        out[mask] = (out[mask] + cur_cell[mask].to(dtype)) / N
        mask = mask & (cur_node != 0)
        if not mask.any():
            break
        packed = parent_depth[cur_node[mask], 0].long()
        cur_cell[mask] = torch.stack(((packed // (N * N)) % N, (packed // N) % N, packed % N), -1)
        cur_node[mask] = packed // (N ** 3)
    return out


def _dda_unit(cen, invdir):
    t1 = -cen * invdir
    t2 = t1 + invdir
    tmin = torch.minimum(t1, t2).max(dim=-1).values.clamp_min(0.0)
    tmax = torch.maximum(t1, t2).min(dim=-1).values.clamp_max(1e9)
    return tmin, tmax


def render(data, child, parent_depth, invradius, offset, origins, dirs, viewdirs, basis_dim,
           step_size=1e-3, background_brightness=1.0, max_steps=100000):
    """(B, 3) colours.  basis_dim <= 0 means RGBA.  Differentiable w.r.t. `data`."""
    N = child.shape[1]
    origins = torch.addcmul(offset, origins, invradius)
    dirs = dirs / dirs.norm(dim=-1, keepdim=True)
    B = dirs.shape[0]
    sh = eval_sh_bases(basis_dim, viewdirs)[:, None] if basis_dim > 0 else None
    invdirs = 1.0 / (dirs + 1e-9)
    t, tmax = _dda_unit(origins, invdirs)
    hit = ~((tmax < 0) | (t > tmax))
    light = torch.ones(B, dtype=data.dtype)
    out = torch.zeros(B, 3, dtype=data.dtype)
    delta_scale = (dirs / invradius[None]).norm(dim=1)
    live = torch.arange(B)[hit & (t < tmax)]
    steps = 0
    while live.numel() and steps < max_steps:
        steps += 1
        pos = origins[live] + t[live, None] * dirs[live]
        vals, node, cell, levels, local = query(data, child, pos, N)
        cube = float(N) ** (-levels.to(data.dtype))
        s0, s1 = _dda_unit(local, invdirs[live])
        delta_t = (s1 - s0) * cube + step_size
        att = torch.exp(-delta_t * torch.relu(vals[:, -1]) * delta_scale[live])
        weight = light[live] * (1.0 - att)
        rgb = vals[:, :-1]
        if basis_dim > 0:
            rgb = torch.sigmoid((sh[live] * rgb.reshape(-1, 3, basis_dim)).sum(-1))
        else:
            rgb = torch.sigmoid(rgb[:, :3])
        out = out.index_add(0, live, weight[:, None] * rgb)
        light = light.index_put((live,), light[live] * att)
        t = t.index_put((live,), t[live] + delta_t.detach())
        live = live[t[live] < tmax[live]]
    out = out + (light * background_brightness)[:, None] * hit[:, None].to(data.dtype)
    out = torch.where(hit[:, None], out, torch.full_like(out, background_brightness))
    return out
