"""GPU parity tests: every HIP kernel, called through the C ABI (ctypes), against
the CPU oracles on the same seeded inputs.  Integer outputs are compared
bit-exactly; float32 outputs to 1e-5 relative (see tests/helpers.py)."""
import math

import pytest
import torch

from crystalformer_amd import hip_funcs, lib, ops
from oracle import kernel_semantics as ks
from oracle import torch_path as tp
from tests.helpers import (ATOL_PROB, RTOL, Problem, assert_close, atol_averages, atol_projected, atol_rows,
                           make_sized_batch, rel_err, to_dev)

pytestmark = pytest.mark.gpu


def enc_fwd_gpu(dev, p, K, W, cutoff, lr, mr, rvlen=True, pairs=False):
    a, rpos, tv, bt, ed, Wd, rv = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, W,
                                         p.rvlen if rvlen else None)
    pr = ops.edge_pairs(p.b.sizes.to(dev)) if pairs else None
    return ops.real_enc_fwd(a, rpos, tv, bt, ed, K, p.dist_max, p.wscale, Wd, rv, cutoff, lr, mr, pairs_u=pr)


def enc_fwd_ref(p, K, W, cutoff, lr, mr):
    return ks.real_enc_fwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, K, p.dist_max, p.wscale, W, p.rvlen,
                           cutoff, lr, mr)


RULES = [(0.0, 2, 0), (-3.5, 2, 2), (-3.5, 1, 0), (5.0, 1, 1)]


def v_atol(p, K, W, cutoff, lr, mr, s_ref=None):
    """Element-wise bound for the value encoding of problem ``p`` (see tests/helpers.py)."""
    T = (2 * lr + 1) ** 3 if cutoff == 0.0 else 4096          # translations per edge (upper bound for adaptive boxes)
    cond = ks.real_enc_fwd_cond(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, K, p.dist_max, p.wscale, p.rvlen,
                                cutoff, lr, mr)
    if W is None:
        return atol_averages(None, cond, T)
    if s_ref is None:
        _, s_ref = enc_fwd_ref(p, K, None, cutoff, lr, mr)
    return atol_projected(s_ref, W, cond, index=p.edges[0], translations=T)


def enc_bwd_atols(p, z_ref, gz, gv, K, W, cutoff, lr, mr, rvlen=True):
    """Element-wise bounds (ga, gW) of the encoding backward: RTOL times the same sums taken over
    the magnitudes of their terms (oracle's magnitude mode, see tests/helpers.py)."""
    ga_mag, gW_mag = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv, K,
                                     p.dist_max, p.wscale, W, p.rvlen if rvlen else None, cutoff, lr, mr,
                                     magnitude=True)
    return RTOL * ga_mag.double(), (None if gW_mag is None else RTOL * gW_mag.double())


@pytest.mark.parametrize("cutoff,lr,mr", RULES)
@pytest.mark.parametrize("H,K,D", [(8, 64, 16), (8, 0, 16), (4, 16, 8), (1, 7, 3), (2, 100, 4), (16, 32, 8)])
def test_real_enc_fwd(dev, H, K, D, cutoff, lr, mr):
    p = Problem([1, 3, 9, 2, 17], H=H, K=K, D=D, seed=21)
    for W in ([p.W, None] if K > 0 else [None]):
        z, v = enc_fwd_gpu(dev, p, K, W, cutoff, lr, mr)
        z_ref, v_ref = enc_fwd_ref(p, K, W, cutoff, lr, mr)
        assert_close(z, z_ref, "z")
        if K > 0:
            assert_close(v, v_ref, "v", atol=v_atol(p, K, W, cutoff, lr, mr))
        else:
            assert v is None


# (fixed cubes of 27 and 125 translations take the short ring of the kernel, 343 the long one)
@pytest.mark.parametrize("cutoff,lr,mr", RULES + [(-3.5, 3, 3), (0.0, 3, 0), (0.0, 1, 0)])
@pytest.mark.parametrize("H,K,D", [(8, 64, 16), (4, 16, 8), (1, 7, 3), (2, 100, 4), (16, 32, 8), (8, 64, 32),
                                   (8, 48, 20), (8, 64, 64), (8, 0, 16), (2, 0, 4)])
def test_real_enc_fwd_pair_kernel(dev, H, K, D, cutoff, lr, mr):
    """Matrix-core path: both directions of an atom pair evaluated together (pair list given)."""
    p = Problem([1, 3, 9, 2, 17, 1], H=H, K=K, D=D, seed=28)
    z_ref, v_ref = enc_fwd_ref(p, K, p.W, cutoff, lr, mr)
    z, v = enc_fwd_gpu(dev, p, K, p.W, cutoff, lr, mr, pairs=True)
    assert_close(z, z_ref, "z")
    if K == 0:                                   # bias only: every translation feeds the column sums
        assert v is None
        return
    _, s_ref = enc_fwd_ref(p, K, None, cutoff, lr, mr)
    assert_close(v, v_ref, "v", atol=v_atol(p, K, p.W, cutoff, lr, mr, s_ref))
    z2, s = enc_fwd_gpu(dev, p, K, None, cutoff, lr, mr, pairs=True)
    assert torch.equal(z2, z) or rel_err(z2, z) < 1e-6
    assert_close(s, s_ref, "s", atol=v_atol(p, K, None, cutoff, lr, mr))


def test_real_enc_pair_kernel_large_boxes_and_indexed_projection(dev):
    """Boxes beyond the staging capacity (several passes per unit) and per-edge / per-atom W."""
    p = Problem([4, 7], H=8, K=64, D=16, seed=29)
    p.a = p.a * 0.05                                  # slow decay -> wide adaptive boxes
    for mr in (0, 4):
        z, v = enc_fwd_gpu(dev, p, 64, p.W, -3.5, 2, mr, pairs=True)
        z_ref, v_ref = enc_fwd_ref(p, 64, p.W, -3.5, 2, mr)
        R = ks.translation_ranges(p.a, p.rvlen, p.b.batch, -3.5, 2, mr)
        assert int((2 * R.max(dim=1).values + 1).prod(dim=1).max()) > 256
        assert_close(z, z_ref, "z")
        assert_close(v, v_ref, "v", atol=v_atol(p, 64, p.W, -3.5, 2, mr))
    for mode in ("edge", "atom"):
        pm = Problem([3, 4, 1], H=4, K=16, D=8, seed=23, W_mode=mode)
        z, v = enc_fwd_gpu(dev, pm, 16, pm.W, -3.5, 2, 2, pairs=True)
        z_ref, v_ref = enc_fwd_ref(pm, 16, pm.W, -3.5, 2, 2)
        assert_close(z, z_ref, "z")
        assert_close(v, v_ref, "v", atol=v_atol(pm, 16, pm.W, -3.5, 2, 2))


@pytest.mark.parametrize("scale,mr", [(0.03, 2), (0.3, 2), (1.0, 3)])
def test_real_enc_pair_kernel_large_boxes_with_the_nearest_image_outside_the_cube(dev, scale, mr):
    """Atoms displaced by whole lattice vectors under the floored rule: every box holds the cube, but the
    nearest image of an edge lies up to four cells away, outside it.  Boxes of several staging passes
    take their reference distance from the cube: weights above 1 (wide Gaussians) or, where that would
    go too far (narrow Gaussians in boxes that a floor of 3 makes large: |a| d2 of the cube's nearest
    image beyond the kernel's limit for many pairs), the pass over the whole box."""
    p = Problem([5, 2, 8, 1], H=8, K=64, D=16, seed=47)
    g = torch.Generator().manual_seed(78)
    shift = torch.randint(-2, 3, (p.N, 3), generator=g).float()
    p.b.pos = p.b.pos + (shift[:, None, :] @ p.b.trans_vec[p.b.batch]).squeeze(1)
    p.rpos = tp.relative_positions(p.b.pos, p.edges)
    p.a = p.a * scale
    R = ks.translation_ranges(p.a, p.rvlen, p.b.batch, -3.5, 2, mr)
    assert int((2 * R.max(dim=1).values + 1).prod(dim=1).max()) > 192
    z_ref, v_ref = enc_fwd_ref(p, 64, p.W, -3.5, 2, mr)
    z, v = enc_fwd_gpu(dev, p, 64, p.W, -3.5, 2, mr, pairs=True)
    ok = torch.isfinite(z_ref)
    assert ok.float().mean() > 0.5
    okv = ok[:, :, None].expand_as(v_ref)
    assert_close(torch.where(ok, z.cpu(), torch.zeros(())), torch.where(ok, z_ref, torch.zeros(())), "z")
    assert_close(torch.where(okv, v.cpu(), torch.zeros(())), torch.where(okv, v_ref, torch.zeros(())), "v")


@pytest.mark.parametrize("scale,mr", [(0.05, 2), (0.05, 0), (0.3, 2), (1.0, 3)])
def test_real_enc_pair_kernels_one_box_for_all_columns(dev, scale, mr):
    """The same exponent for every (atom, head): all 16 columns of an atom pair have one box, which
    is not the cube (wide Gaussians: several staging passes per pair; floor above lattice_range:
    one pass).  The kernels then skip the per-column tables and masks and, for boxes of several
    passes, take the reference distance from the cube."""
    p = Problem([4, 7, 1, 2], H=8, K=64, D=16, seed=43)
    p.a = torch.full_like(p.a, float(p.a.mean()) * scale)
    R = ks.translation_ranges(p.a, p.rvlen, p.b.batch, -3.5, 2, mr)
    assert bool((R == R[:, :1, :]).all())                               # one box per crystal
    T = (2 * R[:, 0, :] + 1).prod(dim=1)
    assert int(T.max()) > (192 if scale < 0.1 else 125)
    z_ref, v_ref = enc_fwd_ref(p, 64, p.W, -3.5, 2, mr)
    z, v = enc_fwd_gpu(dev, p, 64, p.W, -3.5, 2, mr, pairs=True)
    assert_close(z, z_ref, "z")
    assert_close(v, v_ref, "v", atol=v_atol(p, 64, p.W, -3.5, 2, mr))
    gz, gv = p.randn(p.E, 8), p.randn(p.E, 8, 16)
    args = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv)
    ga, gW = ops.real_enc_bwd(*args, 64, p.dist_max, p.wscale, p.W.to(dev), p.rvlen.to(dev), -3.5, 2, mr,
                              pairs_u=ops.edge_pairs(p.b.sizes.to(dev)))
    ga_ref, gW_ref = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv, 64,
                                     p.dist_max, p.wscale, p.W, p.rvlen, -3.5, 2, mr)
    ga_atol, gW_atol = enc_bwd_atols(p, z_ref, gz, gv, 64, p.W, -3.5, 2, mr)
    assert_close(ga, ga_ref, "ga", atol=ga_atol)
    assert_close(gW, gW_ref, "gW", atol=gW_atol)


def test_real_enc_pair_kernels_where_the_sigma_rule_hits_whole_numbers(dev):
    """Exponents chosen so that (3.5 sigma + 0.01) |b| / 2 pi of one axis is a whole number to within a
    few float ulps, per (atom, head): the pair kernels work the half-widths out with one-ulp
    reciprocals and square roots and must fall back to the exact rule there.  A half-width that is off
    by one adds or drops a shell of translations at 3.5 sigma, 2e-3 of the leading term."""
    p = Problem([3, 6, 2], H=8, K=64, D=16, seed=41)
    g = torch.Generator().manual_seed(3)
    two_pi = 2.0 * float(torch.tensor(3.141592654, dtype=torch.float32))
    rv = p.rvlen[p.b.batch].double()                                    # (N, 3)
    axis = torch.randint(0, 3, (p.N, 8), generator=g)
    k = torch.randint(2, 5, (p.N, 8), generator=g).double()
    sigma = (k * two_pi / rv.gather(1, axis) - float(torch.tensor(0.01, dtype=torch.float32))) / 3.5
    a = (-0.5 / (sigma * sigma)).float()
    for _ in range(int(torch.randint(0, 3, (1,), generator=g))):        # a few ulps either way for some
        a = torch.where(torch.rand(p.N, 8, generator=g) < 0.5, torch.nextafter(a, torch.zeros(())), a)
    p.a = a
    R = ks.translation_ranges(p.a, p.rvlen, p.b.batch, -3.5, 2, 0)
    on_axis = R.gather(2, axis[:, :, None]).squeeze(2).double()
    assert float(((on_axis - k).abs() <= 1).float().mean()) == 1.0 and len(set(on_axis.flatten().tolist())) >= 3
    z_ref, v_ref = enc_fwd_ref(p, 64, p.W, -3.5, 2, 0)
    z, v = enc_fwd_gpu(dev, p, 64, p.W, -3.5, 2, 0, pairs=True)
    assert_close(z, z_ref, "z")
    assert_close(v, v_ref, "v", atol=v_atol(p, 64, p.W, -3.5, 2, 0))
    gz, gv = p.randn(p.E, 8), p.randn(p.E, 8, 16)
    args = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv)
    ga, gW = ops.real_enc_bwd(*args, 64, p.dist_max, p.wscale, p.W.to(dev), p.rvlen.to(dev), -3.5, 2, 0,
                              pairs_u=ops.edge_pairs(p.b.sizes.to(dev)))
    ga_ref, gW_ref = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv, 64,
                                     p.dist_max, p.wscale, p.W, p.rvlen, -3.5, 2, 0)
    ga_atol, gW_atol = enc_bwd_atols(p, z_ref, gz, gv, 64, p.W, -3.5, 2, 0)
    assert_close(ga, ga_ref, "ga", atol=ga_atol)
    assert_close(gW, gW_ref, "gW", atol=gW_atol)


@pytest.mark.parametrize("cutoff,mr", [(-3.5, 0), (-1.0, 0), (2.0, 0), (-3.5, 1)])
def test_real_enc_pair_kernel_atoms_outside_the_home_cell(dev, cutoff, mr):
    """Atoms displaced by whole lattice vectors: the nearest image of an edge is then a
    translation n != 0 that small per-column boxes do not contain, so columns of one unit
    have different minimum distances (and some boxes miss the neighbourhood entirely)."""
    p = Problem([5, 2, 8, 1], H=8, K=64, D=16, seed=31)
    g = torch.Generator().manual_seed(77)
    shift = torch.randint(-2, 3, (p.N, 3), generator=g).float()
    p.b.pos = p.b.pos + (shift[:, None, :] @ p.b.trans_vec[p.b.batch]).squeeze(1)
    p.rpos = tp.relative_positions(p.b.pos, p.edges)
    p.a = p.a * torch.linspace(0.3, 3.0, 8)[None, :]        # heads with very different boxes
    z_ref, v_ref = enc_fwd_ref(p, 64, p.W, cutoff, 2, mr)
    z, v = enc_fwd_gpu(dev, p, 64, p.W, cutoff, 2, mr, pairs=True)
    ok = torch.isfinite(z_ref)
    assert ok.float().mean() > 0.5
    assert_close(torch.where(ok, z.cpu(), torch.zeros(())), torch.where(ok, z_ref, torch.zeros(())), "z")
    okv = ok[:, :, None].expand_as(v_ref)
    assert_close(torch.where(okv, v.cpu(), torch.zeros(())), torch.where(okv, v_ref, torch.zeros(())), "v")
    # backward on the same problem
    a, rpos, tv, bt, ed, W, rv, es = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.W, p.rvlen,
                                            p.e_start)
    gz, gv = p.randn(p.E, 8), p.randn(p.E, 8, 16)
    gz = torch.where(ok, gz, torch.zeros(()))
    gv = torch.where(okv, gv, torch.zeros(()))
    pairs = ops.edge_pairs(p.b.sizes.to(dev))
    ga, gW = ops.real_enc_bwd(a, rpos, tv, bt, ed, es, z, gz.to(dev), gv.to(dev), 64, p.dist_max, p.wscale, W, rv,
                              cutoff, 2, mr, pairs_u=pairs)
    ga_ref, gW_ref = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv, 64,
                                     p.dist_max, p.wscale, p.W, p.rvlen, cutoff, 2, mr)
    if bool(ok.all()):
        # exp(a d^2 - z) with |a d^2| ~ |z| ~ 10^3 here: the difference of two such float32 numbers
        # carries ~1e-4 absolute error whatever the summation order, so this (deliberately extreme)
        # case is held to 1e-4 instead of 1e-5
        assert_close(ga, ga_ref, "ga", rtol=1e-4)
        assert_close(gW, gW_ref.reshape(gW.shape), "gW", rtol=1e-4)


@pytest.mark.parametrize("cutoff,lr,mr", RULES[:3] + [(0.0, 3, 0)])
@pytest.mark.parametrize("H,K,D", [(8, 64, 16), (4, 16, 8), (16, 32, 16), (1, 7, 12), (8, 64, 32)])
def test_real_enc_bwd_pair_kernel(dev, H, K, D, cutoff, lr, mr):
    p = Problem([1, 3, 9, 2, 14, 1, 1, 1, 1, 20], H=H, K=K, D=D, seed=30)
    z_ref, v_ref = enc_fwd_ref(p, K, p.W, cutoff, lr, mr)
    gz, gv = p.randn(p.E, H), p.randn(*v_ref.shape)
    args = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv)
    pairs = ops.edge_pairs(p.b.sizes.to(dev))
    ga, gW = ops.real_enc_bwd(*args, K, p.dist_max, p.wscale, p.W.to(dev), p.rvlen.to(dev), cutoff, lr, mr,
                              pairs_u=pairs)
    ga_ref, gW_ref = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv, K,
                                     p.dist_max, p.wscale, p.W, p.rvlen, cutoff, lr, mr)
    ga_atol, gW_atol = enc_bwd_atols(p, z_ref, gz, gv, K, p.W, cutoff, lr, mr)
    assert_close(ga, ga_ref, "ga", atol=ga_atol)
    assert_close(gW, gW_ref, "gW", atol=gW_atol)
    # without the gradient of W
    ga2, none = ops.real_enc_bwd(*args, K, p.dist_max, p.wscale, p.W.to(dev), p.rvlen.to(dev), cutoff, lr, mr,
                                 want_gW=False, pairs_u=pairs)
    assert none is None and torch.equal(ga2, ga)


def test_pair_kernels_are_bit_stable(dev):
    """No atomics: repeated launches give identical bits, forward and backward."""
    p = Problem([5, 11, 2, 30], H=8, K=64, D=16, seed=31)
    pairs = ops.edge_pairs(p.b.sizes.to(dev))
    a, rpos, tv, bt, ed, W, rv, es = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.W, p.rvlen,
                                            p.e_start)
    runs = [ops.real_enc_fwd(a, rpos, tv, bt, ed, 64, p.dist_max, 1.0, W, rv, -3.5, 2, 2, pairs_u=pairs)
            for _ in range(3)]
    assert all(torch.equal(r[0], runs[0][0]) and torch.equal(r[1], runs[0][1]) for r in runs)
    z, v = runs[0]
    gz, gv = p.randn(p.E, 8).to(dev), p.randn(p.E, 8, 16).to(dev)
    bruns = [ops.real_enc_bwd(a, rpos, tv, bt, ed, es, z, gz, gv, 64, p.dist_max, 1.0, W, rv, -3.5, 2, 2,
                              pairs_u=pairs) for _ in range(3)]
    assert all(torch.equal(r[0], bruns[0][0]) and torch.equal(r[1], bruns[0][1]) for r in bruns)


def test_edge_pairs_bit_exact(dev):
    for sizes in ([1], [3, 1, 4, 1, 5], [64, 1, 33]):
        b = make_sized_batch(sizes, seed=45)
        pairs = ops.edge_pairs(b.sizes.to(dev)).cpu()
        edges = tp.get_edge_index(sizes)
        ref, aoff, eoff = [], 0, 0
        for b_idx, n in enumerate(sizes):
            for i in range(n):
                for j in range(i, n):
                    ref.append((eoff + i * n + j, eoff + j * n + i, aoff + i, aoff + j, b_idx))
            eoff += n * n
            aoff += n
        assert pairs.dtype == torch.int64 and pairs.tolist() == [list(r) for r in ref]
        assert torch.equal(edges[0][pairs[:, 0]], edges[1][pairs[:, 1]])
        assert torch.equal(edges[0][pairs[:, 0]], pairs[:, 2]) and torch.equal(edges[1][pairs[:, 0]], pairs[:, 3])
        assert torch.equal(b.batch[pairs[:, 2]], pairs[:, 4])


def test_real_enc_fwd_matches_torch_path_fixed_cube(dev):
    """Against the reference's PyTorch-path semantics (dense (E,R) tensors)."""
    p = Problem([2, 5, 1, 12], H=8, K=64, D=16, seed=22)
    for r in (1, 2):
        z, v = enc_fwd_gpu(dev, p, 64, p.W, 0.0, r, 0, rvlen=False)
        z_ref, v_ref = tp.periodic_encoding(p.a, p.b.pos, p.b.batch, p.b.trans_vec, p.edges, r, 64, p.dist_max,
                                            p.wscale, p.W)
        _, s_ref = tp.periodic_encoding(p.a, p.b.pos, p.b.batch, p.b.trans_vec, p.edges, r, 64, p.dist_max,
                                        p.wscale, None)
        assert_close(z, z_ref, "z")
        cond = ks.real_enc_fwd_cond(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, 64, p.dist_max, p.wscale, None,
                                    0.0, r, 0)
        assert_close(v, v_ref, "v", atol=atol_projected(s_ref, p.W, cond, translations=(2 * r + 1) ** 3))


@pytest.mark.parametrize("mode", ["edge", "atom"])
def test_real_enc_indexed_projection(dev, mode):
    p = Problem([3, 4, 1], H=4, K=16, D=8, seed=23, W_mode=mode)
    z, v = enc_fwd_gpu(dev, p, 16, p.W, -3.5, 2, 2)
    z_ref, v_ref = enc_fwd_ref(p, 16, p.W, -3.5, 2, 2)
    _, s_ref = enc_fwd_ref(p, 16, None, -3.5, 2, 2)
    assert_close(z, z_ref, "z")
    assert_close(v, v_ref, "v", atol=v_atol(p, 16, p.W, -3.5, 2, 2, s_ref))
    gz, gv = p.randn(p.E, 4), p.randn(p.E, 4, 8)
    args = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv)
    ga, gW = ops.real_enc_bwd(*args, 16, p.dist_max, p.wscale, p.W.to(dev), p.rvlen.to(dev), -3.5, 2, 2)
    ga_ref, gW_ref = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv, 16,
                                     p.dist_max, p.wscale, p.W, p.rvlen, -3.5, 2, 2)
    ga_atol, gW_atol = enc_bwd_atols(p, z_ref, gz, gv, 16, p.W, -3.5, 2, 2)
    assert_close(ga, ga_ref, "ga", atol=ga_atol)
    assert_close(gW, gW_ref, "gW", atol=gW_atol)


@pytest.mark.parametrize("cutoff,lr,mr", RULES[:3])
@pytest.mark.parametrize("H,K,D", [(8, 64, 16), (8, 0, 16), (4, 16, 8), (2, 100, 4)])
def test_real_enc_bwd(dev, H, K, D, cutoff, lr, mr):
    p = Problem([1, 3, 9, 2, 14], H=H, K=K, D=D, seed=24)
    for W in ([p.W, None] if K > 0 else [None]):
        z_ref, v_ref = enc_fwd_ref(p, K, W, cutoff, lr, mr)
        gz = p.randn(p.E, H)
        gv = p.randn(*v_ref.shape) if K > 0 else None
        args = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv)
        ga, gW = ops.real_enc_bwd(*args, K, p.dist_max, p.wscale, None if W is None else W.to(dev),
                                  p.rvlen.to(dev), cutoff, lr, mr)
        ga_ref, gW_ref = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv,
                                         K, p.dist_max, p.wscale, W, p.rvlen, cutoff, lr, mr)
        ga_atol, gW_atol = enc_bwd_atols(p, z_ref, gz, gv, K, W, cutoff, lr, mr)
        assert_close(ga, ga_ref, "ga", atol=ga_atol)
        if W is not None:
            assert_close(gW, gW_ref, "gW", atol=gW_atol)
        else:
            assert gW is None


def test_real_enc_bwd_without_value_gradient(dev):
    p = Problem([4, 2], H=8, K=64, D=16, seed=25)
    z_ref, _ = enc_fwd_ref(p, 64, p.W, 0.0, 2, 0)
    gz = p.randn(p.E, 8)
    args = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, None)
    ga, gW = ops.real_enc_bwd(*args, 64, p.dist_max, p.wscale, p.W.to(dev), None, 0.0, 2, 0)
    ga_ref, _ = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, None, 64,
                                p.dist_max, p.wscale, p.W, None, 0.0, 2, 0)
    assert_close(ga, ga_ref, "ga")
    assert float(gW.abs().max()) == 0.0


@pytest.mark.parametrize("cutoff,lr,mr", [(0.0, 2, 0), (-3.5, 2, 2), (-3.5, 2, 0), (4.0, 1, 0), (-1.0, 3, 1)])
def test_translation_ranges_bit_exact(dev, cutoff, lr, mr):
    p = Problem([5, 9, 1, 30], H=8, K=0, seed=26)
    a = p.a * torch.logspace(-1.5, 1.0, p.N)[:, None]            # spread the exponents over decades
    got = ops.translation_ranges(a.to(dev), p.rvlen.to(dev), p.b.batch.to(dev), cutoff, lr, mr).cpu()
    ref = ks.translation_ranges(a, p.rvlen, p.b.batch, cutoff, lr, mr)
    assert got.dtype == torch.int32 and torch.equal(got, ref)


def test_translation_ranges_at_integer_quotients(dev):
    """Half-widths where (cutoff + 0.01) * |b| / 2 pi sits on, or within a few float ulps of, an
    integer: the ceiling must come from the double quotient there (the kernel only takes its float
    shortcut away from integers)."""
    two_pi = 2.0 * float(torch.tensor(3.141592654, dtype=torch.float32))
    cutoff = 3.0
    ks_int = torch.arange(1, 41, dtype=torch.float64)
    base = (ks_int * two_pi / (float(torch.tensor(cutoff, dtype=torch.float32)) + float(torch.tensor(0.01, dtype=torch.float32)))).float()
    variants = [base]
    for _ in range(3):
        variants.append(torch.nextafter(variants[-1], torch.full_like(base, 1e9)))
    lo = base
    for _ in range(3):
        lo = torch.nextafter(lo, torch.zeros_like(base))
        variants.append(lo)
    rv = torch.stack(variants).reshape(-1)                      # 280 reciprocal lengths
    B = rv.numel()
    rvlen = torch.stack([rv, rv.flip(0), rv.roll(7)], dim=1).contiguous()
    batch = torch.arange(B)
    a = -torch.rand(B, 8, generator=torch.Generator().manual_seed(2)) - 0.1
    for mr in (0, 2):
        got = ops.translation_ranges(a.to(dev), rvlen.to(dev), batch.to(dev), cutoff, 2, mr).cpu()
        ref = ks.translation_ranges(a, rvlen, batch, cutoff, 2, mr)
        assert torch.equal(got, ref)
    assert int(ref.max()) >= 40 and len(set(ref[:, 0, 0].tolist())) > 30


def test_empty_and_single_atom_inputs(dev):
    # no crystals at all
    z, v = ops.real_enc_fwd(torch.zeros(0, 8, device=dev), torch.zeros(0, 3, device=dev),
                            torch.zeros(0, 3, 3, device=dev), torch.zeros(0, dtype=torch.long, device=dev),
                            torch.zeros(2, 0, dtype=torch.long, device=dev), 64, 14.0, 1.0,
                            torch.zeros(1, 8, 16, 64, device=dev))
    assert z.shape == (0, 8) and v.shape == (0, 8, 16)
    e, r = ops.edge_index(torch.zeros(0, dtype=torch.long, device=dev), torch.zeros(0, 3, device=dev))
    assert e.shape == (2, 0) and r.shape == (0, 3)
    # crystals of one atom: a single self edge with r_ij = 0
    p = Problem([1, 1, 1], H=8, K=64, D=16, seed=27)
    z, v = enc_fwd_gpu(dev, p, 64, p.W, 0.0, 2, 0, rvlen=False)
    z_ref, v_ref = enc_fwd_ref(p, 64, p.W, 0.0, 2, 0)
    assert_close(z, z_ref, "z")
    assert_close(v, v_ref, "v")
    assert bool((z.cpu() >= 0).all())      # the n = 0 term alone contributes exp(0) = 1


# ------------------------------------------------------------ fused attention
def dpa_problem(sizes, H, Dk, Dv, seed, bias=True, vals=True):
    p = Problem(sizes, H=H, K=0, seed=seed)
    q = p.randn(p.N, H, Dk) / math.sqrt(Dk)
    k, v = p.randn(p.N, H, Dk), p.randn(p.N, H, Dv)
    a = p.randn(p.E, H) * 2 if bias else None
    b = p.randn(p.E, H, Dv) if vals else None
    return p, q, k, v, a, b


def dpa_atols(p, q, k, v, b, prob, out):
    """Element-wise bounds for the attention (see tests/helpers.py): every output entry is a sum
    over the edges of a row or column; its bound is RTOL times the sum of the magnitudes of the
    terms, formed here from the oracle's probabilities."""
    i, j = p.edges
    P = prob.double()
    msg = v.double()[j] if b is None else v.double()[j] + b.double()
    out_atol = RTOL * torch.zeros_like(out, dtype=torch.float64).index_add_(0, i, P[..., None] * msg.abs())

    def backward_bounds(go):
        g = go.double()[i]                                               # (E,H,Dv)
        t = P[..., None] * g.abs()                                       # |gb| terms
        dev_ = msg.abs() + out.double()[i].abs()                        # |v_j + b_ij| + |o_i|: the two are subtracted
        gs_abs = (dev_ * t).sum(-1)                                      # sum_d |(v_j + b - o_i)_d go_d p|
        N = q.shape[0]
        zq = torch.zeros(q.shape, dtype=torch.float64)
        zv = torch.zeros(v.shape, dtype=torch.float64)
        return dict(gq=RTOL * zq.clone().index_add_(0, i, gs_abs[..., None] * k.double()[j].abs()),
                    gk=RTOL * zq.clone().index_add_(0, j, gs_abs[..., None] * q.double()[i].abs()),
                    gv=RTOL * zv.clone().index_add_(0, j, t),
                    gaij=RTOL * gs_abs, gbij=1e-37)
    return out_atol, backward_bounds


@pytest.mark.parametrize("bias,vals", [(True, True), (True, False), (False, False), (False, True)])
@pytest.mark.parametrize("H,Dk,Dv,sizes", [(8, 16, 16, [1, 5, 70, 2, 33]), (4, 8, 32, [3, 65]), (1, 5, 4, [7, 2]),
                                           (16, 16, 16, [9, 1]), (2, 64, 64, [4]),
                                           (8, 16, 16, [32, 64, 31, 8]),      # rows of exactly one and two whole steps
                                           (4, 8, 8, [17, 40]), (2, 4, 4, [130]), (1, 32, 32, [12]),
                                           (8, 16, 16, [200, 150, 97]),       # long rows: the prefetching variant
                                           (8, 16, 16, [70, 66, 65])])
def test_fused_dpa_fwd_bwd(dev, H, Dk, Dv, sizes, bias, vals):
    p, q, k, v, a, b = dpa_problem(sizes, H, Dk, Dv, 31, bias, vals)
    out, prob = ops.fused_dpa_fwd(*to_dev(dev, q, k, v, a, b, p.edges, p.e_start))
    out_ref, prob_ref = ks.fused_dpa_fwd(q, k, v, a, b, p.edges, p.e_start)
    out_atol, bounds = dpa_atols(p, q, k, v, b, prob_ref, out_ref)
    assert_close(out, out_ref, "out", atol=out_atol)
    assert_close(prob, prob_ref, "prob", atol=ATOL_PROB)
    go = p.randn(p.N, H, Dv)
    got = ops.fused_dpa_bwd(*to_dev(dev, q, k, v, b, p.b.batch, p.edges, p.e_start, prob_ref, out_ref, go))
    ref = ks.fused_dpa_bwd(q, k, v, b, p.edges, p.e_start, prob_ref, out_ref, go)
    atols = bounds(go)
    for name, x, y in zip(("gq", "gk", "gv", "gaij", "gbij"), got, ref):
        if y is None:
            assert x is None
        else:
            assert_close(x, y, name, atol=atols[name])


@pytest.mark.parametrize("H,D", [(8, 16), (1, 5)])
def test_fused_dpa_fwd_on_an_arbitrary_edge_list(dev, H, D):
    """The forward takes any edge list sorted by source atom: a random third of the dense edges
    removed, one atom left without any edge (its output row is zero)."""
    p, q, k, v, a, b = dpa_problem([5, 40, 70, 3], H, D, D, 35)
    gen = torch.Generator().manual_seed(3)
    keep = torch.rand(p.E, generator=gen) > 0.33
    keep &= p.edges[0] != 17                                   # atom 17 loses every edge
    edges = p.edges[:, keep].contiguous()
    e_start = tp.edge_row_offsets(edges, p.N)
    a, b = a[keep].contiguous(), b[keep].contiguous()
    out, prob = ops.fused_dpa_fwd(*to_dev(dev, q, k, v, a, b, edges, e_start))
    out_ref, prob_ref = ks.fused_dpa_fwd(q, k, v, a, b, edges, e_start)
    assert_close(out, out_ref, "out")
    assert_close(prob, prob_ref, "prob")
    assert float(out[17].abs().max()) == 0.0
    rows = torch.zeros(p.N, H).index_add_(0, edges[0], prob.cpu())
    has = (e_start[1:] - e_start[:-1]) > 0
    assert not bool(has[17]) and int(has.sum()) > p.N // 2
    assert float((rows[has] - 1.0).abs().max()) < 1e-5         # each row's weights sum to one
    assert float(out.cpu()[~has].abs().max()) == 0.0


@pytest.mark.parametrize("H,D,sizes", [(8, 16, [70, 90, 3, 130, 1, 101]), (4, 16, [150, 5, 160, 137]),
                                       (16, 16, [33, 70, 2, 45]), (8, 8, [150, 131, 7, 160]),
                                       (2, 32, [130, 171, 1])])
@pytest.mark.parametrize("bias,vals", [(True, True), (False, True), (True, False), (False, False)])
def test_fused_dpa_fwd_long_rows(dev, H, D, sizes, bias, vals):
    """Rows longer than two steps of a work-group on average take the variant that keeps the key
    indices a step ahead and every load of a step in flight: lane layouts of 16, 32 and 64 lanes per
    edge, crystals whose sizes are no multiple of a step (single-atom crystals between long ones),
    with and without a_ij / b_ij."""
    p, q, k, v, a, b = dpa_problem(sizes, H, D, D, 36, bias, vals)
    assert p.E > 2 * (16 * 64 // (H * D // 4)) * p.N            # the launch rule for long rows
    out, prob = ops.fused_dpa_fwd(*to_dev(dev, q, k, v, a, b, p.edges, p.e_start))
    out_ref, prob_ref = ks.fused_dpa_fwd(q, k, v, a, b, p.edges, p.e_start)
    out_atol, _ = dpa_atols(p, q, k, v, b, prob_ref, out_ref)
    assert_close(out, out_ref, "out", atol=out_atol)
    assert_close(prob, prob_ref, "prob", atol=ATOL_PROB)


def test_fused_dpa_fwd_long_rows_on_an_arbitrary_edge_list(dev):
    """The same variant on an edge list that is no dense block (a random fifth of the edges removed,
    one atom without edges)."""
    p, q, k, v, a, b = dpa_problem([120, 150, 90], 8, 16, 16, 37)
    gen = torch.Generator().manual_seed(6)
    keep = torch.rand(p.E, generator=gen) > 0.2
    keep &= p.edges[0] != 133
    edges = p.edges[:, keep].contiguous()
    e_start = tp.edge_row_offsets(edges, p.N)
    a, b = a[keep].contiguous(), b[keep].contiguous()
    assert edges.shape[1] > 2 * 32 * p.N
    out, prob = ops.fused_dpa_fwd(*to_dev(dev, q, k, v, a, b, edges, e_start))
    out_ref, prob_ref = ks.fused_dpa_fwd(q, k, v, a, b, edges, e_start)
    assert_close(out, out_ref, "out")
    assert_close(prob, prob_ref, "prob", atol=ATOL_PROB)
    assert float(out[133].abs().max()) == 0.0


def test_fused_dpa_beyond_the_reference_size_limit(dev):
    """The reference's kernels stop at 320 atoms per crystal; these do not."""
    p, q, k, v, a, b = dpa_problem([444, 3], 8, 16, 16, 32)
    out, prob = ops.fused_dpa_fwd(*to_dev(dev, q, k, v, a, b, p.edges, p.e_start))
    out_ref, prob_ref = ks.fused_dpa_fwd(q, k, v, a, b, p.edges, p.e_start)
    out_atol, bounds = dpa_atols(p, q, k, v, b, prob_ref, out_ref)
    assert_close(out, out_ref, "out", atol=out_atol)
    assert_close(prob, prob_ref, "prob", atol=ATOL_PROB)
    go = p.randn(p.N, 8, 16)
    got = ops.fused_dpa_bwd(*to_dev(dev, q, k, v, b, p.b.batch, p.edges, p.e_start, prob_ref, out_ref, go))
    ref = ks.fused_dpa_bwd(q, k, v, b, p.edges, p.e_start, prob_ref, out_ref, go)
    atols = bounds(go)
    for name, x, y in zip(("gq", "gk", "gv", "gaij", "gbij"), got, ref):
        assert_close(x, y, name, atol=atols[name])


def test_fused_dpa_large_logits_are_stable(dev):
    p, q, k, v, a, b = dpa_problem([20], 8, 16, 16, 33)
    a = a * 200.0                                   # logits of +-1000: max-subtraction must hold
    out, prob = ops.fused_dpa_fwd(*to_dev(dev, q, k, v, a, b, p.edges, p.e_start))
    out_ref, prob_ref = ks.fused_dpa_fwd(q, k, v, a, b, p.edges, p.e_start)
    assert_close(out, out_ref, "out", atol=dpa_atols(p, q, k, v, b, prob_ref, out_ref)[0])
    # a logit of 1000 carries 1000 * 2^-24 = 6e-5 of float32 rounding before the exponential:
    # the weights are held to that, not to 1e-5 of themselves
    assert_close(prob, prob_ref, "prob")
    assert float(((prob.cpu() - prob_ref).abs() / prob_ref.clamp_min(1e-12)).max()) < 2e-4


# ------------------------------------------------------------ irregular ops
@pytest.mark.parametrize("sizes,D", [([1, 5, 70, 2], 128), ([1500, 3], 7), ([2], 1)])
def test_irregular_mean(dev, sizes, D):
    b = make_sized_batch(sizes, seed=41)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(int(b.sizes.sum()), D, generator=g) + 3.0
    start = tp.crystal_starts(b.sizes)
    got = ops.irregular_mean_fwd(x.to(dev), start.to(dev))
    assert_close(got, ks.irregular_mean(x, start), "mean")
    assert_close(got, tp.avr_pool(x.double(), b.sizes).float(), "mean vs torch")
    go = torch.randn(len(sizes), D, generator=g)
    gx = ops.irregular_mean_bwd(go.to(dev), b.batch.to(dev), start.to(dev))
    ref = (go / b.sizes.view(-1, 1).float())[b.batch]
    assert_close(gx, ref, "mean bwd")


def test_get_edge_index_by_the_reference_name(dev):
    """encoder.get_edge_index(sizes, device): the reference's host function
    (models/indexed_latticeformer_encoder.py:15-32) served by the device kernel, from a list or a
    tensor of sizes, crystals without atoms included."""
    from crystalformer_amd.encoder import get_edge_index
    for sizes in ([3, 1, 4], [2, 0, 5, 0], [7]):
        ref = tp.get_edge_index(sizes)
        assert torch.equal(get_edge_index(sizes, dev).cpu(), ref)
        assert torch.equal(get_edge_index(torch.tensor(sizes), dev).cpu(), ref)
    assert get_edge_index([], dev).shape == (2, 0) and get_edge_index([0, 0], dev).shape == (2, 0)


@pytest.mark.parametrize("sizes", [[1], [3, 1, 4, 1, 5], [64, 1, 33], [200]])
def test_edge_index_bit_exact(dev, sizes):
    b = make_sized_batch(sizes, seed=42)
    edges, rpos = ops.edge_index(b.sizes.to(dev), b.pos.to(dev))
    ref = tp.get_edge_index(sizes)
    assert edges.dtype == torch.int64 and torch.equal(edges.cpu(), ref)
    assert torch.equal(rpos.cpu(), tp.relative_positions(b.pos, ref))      # one subtraction: bit-exact
    assert torch.equal(ops.edge_row_offsets(edges, b.pos.shape[0]).cpu(), tp.edge_row_offsets(ref, b.pos.shape[0]))
    atom_start, edge_start = ops.crystal_offsets(b.batch.to(dev))
    B = len(sizes)
    assert torch.equal(atom_start[:B + 1].cpu(), tp.crystal_starts(b.sizes))
    assert torch.equal(edge_start[:B + 1].cpu(), tp.crystal_starts(b.sizes * b.sizes))


def test_minimum_distance(dev):
    p = Problem([3, 8, 1], H=1, K=0, seed=43)
    for cutoff, lr, mr in [(0.0, 2, 0), (6.0, 1, 0), (2.0, 1, 2)]:
        got = ops.minimum_distance(*to_dev(dev, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.rvlen), cutoff, lr, mr)
        ref = ks.minimum_distance(p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.rvlen, cutoff, lr, mr)
        assert_close(got, ref, "d2min")


def test_errors_surface_as_exceptions(dev):
    p = Problem([2], H=3, K=0, seed=44)           # three heads: not an instantiated width
    with pytest.raises(lib.CrystalformerHipError, match="head count"):
        enc_fwd_gpu(dev, p, 0, None, 0.0, 2, 0)
    p = Problem([2], H=8, K=64, seed=44)
    with pytest.raises(lib.CrystalformerHipError):
        ops.real_enc_fwd(p.a.to(dev), p.rpos.to(dev).double(), p.b.trans_vec.to(dev), p.b.batch.to(dev),
                         p.edges.to(dev), 64, 14.0, 1.0, p.W.to(dev))


def test_lattice_geometry(dev):
    """Cell volume bit-exact with the un-contracted elementwise expression; reciprocal
    vectors and their lengths to float32 rounding."""
    g = torch.Generator().manual_seed(5)
    trans = torch.randn(257, 3, 3, generator=g) * 4 + torch.eye(3) * 6
    vcell, recip, rvlen = ops.lattice_geometry(trans.to(dev))
    rec_ref, v_ref = tp.reciprocal_vectors(trans)
    assert torch.equal(vcell.cpu(), v_ref)
    assert_close(recip, rec_ref, "recip", rtol=1e-6)
    assert_close(rvlen, rec_ref.norm(dim=-1), "rvlen", rtol=1e-6)
    # closed form: rows of recip are dual to the lattice rows, b_r . a_c = 2 pi delta_rc
    dual = torch.einsum("brk,bck->brc", recip.cpu().double(), trans.double())
    assert (dual - 2 * math.pi * torch.eye(3, dtype=torch.float64)).abs().max() < 1e-4


@pytest.mark.parametrize("N,H,D", [(1900, 8, 16), (3, 1, 5), (57000, 8, 16), (33, 16, 8)])
@pytest.mark.parametrize("stored", [False, True])
def test_gauss_exponents(dev, N, H, D, stored):
    g = torch.Generator().manual_seed(N + H)
    q = torch.randn(N, H, D, generator=g) * 1.7 + 0.3
    w = torch.randn(H * D, generator=g) * D ** -0.5
    gs = torch.tensor([1.3, -0.2]) if stored else torch.zeros(2)
    lb, beta, r0 = 0.5, 0.1, 1.4
    gs_ref = gs.clone()
    a_ref = tp.gaussian_exponents(q, w, gs_ref, True, True, lb, beta, r0)
    gs_dev = gs.to(dev)
    a, qs, alpha_n, used = ops.gauss_exponents(q.to(dev), w.to(dev), gs_dev, True, True, "elu", beta, lb,
                                               -0.5 * r0 ** -2, 0.25, want_alpha=True)
    assert_close(a, a_ref, "a")
    assert torch.equal(qs.cpu(), q * 0.25)
    assert_close(gs_dev, gs_ref, "stored statistics")           # written by the training call
    assert_close(used, gs_ref, "statistics used")
    # second call reads the stored pair, inference mode leaves it alone
    before = gs_dev.clone()
    a2, _, _, _ = ops.gauss_exponents(q.to(dev), w.to(dev), gs_dev, True, False, "elu", beta, lb,
                                      -0.5 * r0 ** -2, None)
    assert torch.equal(gs_dev, before)
    assert_close(a2, a_ref, "a from stored statistics")
    # normalised alpha has zero mean / unit std when the batch statistics were used
    if not stored:
        assert abs(float(alpha_n.double().mean())) < 1e-4 and abs(float(alpha_n.double().std()) - 1) < 1e-4


@pytest.mark.parametrize("func", ["elu", "abs", "exp"])
def test_gauss_exponents_positive_maps_and_plain_mode(dev, func):
    from crystalformer_amd.attention import make_positive_func
    g = torch.Generator().manual_seed(3)
    q = torch.randn(40, 4, 12, generator=g)
    w = torch.randn(4, 12, generator=g) * 0.3
    spec = func if func == "abs" else func + "=0.3"
    alpha = (q * w[None]).sum(-1)
    ref = make_positive_func(spec)(alpha, 0.4) * -0.2
    a, qs, _, used = ops.gauss_exponents(q.to(dev), w.to(dev), None, False, False, func, 0.3, 0.4, -0.2)
    assert qs is None and used is None
    assert_close(a, ref, "a")


def test_gauss_exponents_autograd(dev):
    from crystalformer_amd.hip_funcs import GaussianExponentsHIP
    g = torch.Generator().manual_seed(9)
    q = torch.randn(50, 8, 16, generator=g)
    w = torch.randn(128, generator=g) * 0.25
    ga = torch.randn(50, 8, generator=g)
    gqs = torch.randn(50, 8, 16, generator=g)
    qr, wr = q.clone().requires_grad_(), w.clone().requires_grad_()
    a_ref = tp.gaussian_exponents(qr, wr, torch.zeros(2), False, True, 0.5, 0.1, 1.4)
    ((a_ref * ga).sum() + (qr * 0.25 * gqs).sum()).backward()
    qd, wd = q.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    a, qs = GaussianExponentsHIP.apply(qd, wd, torch.zeros(2, device=dev), True, False, "elu", 0.1, 0.5,
                                       -0.5 * 1.4 ** -2, 0.25)
    ((a * ga.to(dev)).sum() + (qs * gqs.to(dev)).sum()).backward()
    assert_close(a, a_ref.detach(), "a")
    assert_close(qd.grad, qr.grad, "gq")
    assert_close(wd.grad, wr.grad, "gw")


def test_batch_layout_bit_exact_and_cached(dev):
    sizes = [3, 1, 4, 1, 5]
    b = make_sized_batch(sizes, seed=3)
    s_dev, bt_dev = b.sizes.to(dev), (b.batch + 7).to(dev)        # batch ids need not start at 0
    lay = ops.batch_layout(s_dev, bt_dev)
    edges = tp.get_edge_index(sizes)
    assert torch.equal(lay.edges.cpu(), edges)
    assert torch.equal(lay.batch.cpu(), b.batch)
    assert torch.equal(lay.e_start.cpu(), tp.edge_row_offsets(edges, b.pos.shape[0]))
    assert (lay.num_atoms, lay.num_edges) == (14, 52)
    assert ops.batch_layout(s_dev, bt_dev) is lay                  # same tensors: cached
    rpos = ops.relative_positions(lay, b.pos.to(dev))
    assert torch.equal(rpos.cpu(), tp.relative_positions(b.pos, edges))
    other = ops.batch_layout(torch.tensor([2, 2], device=dev), torch.tensor([0, 0, 1, 1], device=dev))
    assert other is not lay and other.num_edges == 8
    with pytest.raises(lib.CrystalformerHipError):
        ops.batch_layout(torch.tensor([2, 2], device=dev), torch.tensor([0, 0, 1], device=dev))


@pytest.mark.parametrize("B,hi", [(1, 7), (128, 64), (300, 40), (1000, 9)])
def test_batch_layout_structures_bit_exact(dev, B, hi):
    """Prefix sums, row offsets, edge list and pair list of the one-call layout against the
    oracle's loops and against the operators that build them one by one (more crystals than
    the scan has threads included)."""
    gen = torch.Generator().manual_seed(B)
    sizes = torch.randint(1, hi + 1, (B,), generator=gen)
    batch = torch.repeat_interleave(torch.arange(B), sizes)
    lay = ops.batch_layout(sizes.to(dev), batch.to(dev))
    zero = torch.zeros(1, dtype=torch.long)
    assert torch.equal(lay.atom_start.cpu(), torch.cat([zero, sizes.cumsum(0)]))
    assert torch.equal(lay.edge_start.cpu(), torch.cat([zero, (sizes * sizes).cumsum(0)]))
    edges = tp.get_edge_index(sizes.tolist())
    assert torch.equal(lay.edges.cpu(), edges)
    assert torch.equal(lay.e_start.cpu(), tp.edge_row_offsets(edges, int(sizes.sum())))
    assert torch.equal(lay.pairs, ops.edge_pairs(sizes.to(dev)))
    assert torch.equal(lay.e_start, ops.edge_row_offsets(lay.edges, lay.num_atoms))


@pytest.mark.parametrize("N,K,C,nw", [(1774, 128, 128, 3), (1774, 128, 512, 1), (1774, 512, 128, 1), (5, 16, 7, 2),
                                      (33, 48, 100, 1), (64, 64, 64, 3),
                                      (9000, 128, 128, 3), (9001, 48, 96, 1)])     # beyond 8192 rows: the full-height tiles
def test_linear_rows(dev, N, K, C, nw):
    g = torch.Generator().manual_seed(N + C)
    x = torch.randn(N, K, generator=g)
    ws = [torch.randn(C, K, generator=g) * K ** -0.5 for _ in range(nw)]
    bias = torch.randn(nw * C, generator=g)
    ys = ops.linear_rows(x.to(dev), [w.to(dev) for w in ws], bias.to(dev))
    for i, (w, y) in enumerate(zip(ws, ys)):
        ref = (x.double() @ w.double().T + bias[i * C:(i + 1) * C].double()).float()
        assert_close(y, ref, f"y{i}", rtol=2e-6)
    if nw == 1:
        res = torch.randn(N, C, generator=g)
        y, = ops.linear_rows(x.to(dev), [ws[0].to(dev)], None, residual=res.to(dev), relu=True)
        ref = torch.relu(x.double() @ ws[0].double().T + res.double()).float()
        assert_close(y, ref, "relu(x w^T + r)", rtol=2e-6)
    with pytest.raises(lib.CrystalformerHipError):
        ops.linear_rows(torch.randn(4, 10).to(dev), [torch.randn(3, 10).to(dev)])


@pytest.mark.parametrize("sizes,H", [([256, 256], 8), ([200, 200], 16)])
def test_real_enc_fwd_ticket_rounds_are_bit_identical(dev, sizes, H):
    """Enough units for the shared-counter scheduling to engage (>= 16 rounds per work-group):
    same bits as the fixed stride, scheduling words handed back zeroed, launch after launch."""
    p = Problem(sizes, H=H, K=16, D=8, seed=41)
    a, rpos, tv, bt, ed, W, rv = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.W, p.rvlen)
    pairs = ops.edge_pairs(p.b.sizes.to(dev))
    assert ((pairs.shape[0] + 7) // 8) * ((H + 7) // 8) >= 16 * 512
    for cutoff in (0.0, -3.5):
        ops.DYNAMIC_ROUNDS = False
        try:
            z0, v0 = ops.real_enc_fwd(a, rpos, tv, bt, ed, 16, p.dist_max, 1.0, W, rv, cutoff, 1, 0, pairs_u=pairs)
        finally:
            ops.DYNAMIC_ROUNDS = True
        for _ in range(3):
            z1, v1 = ops.real_enc_fwd(a, rpos, tv, bt, ed, 16, p.dist_max, 1.0, W, rv, cutoff, 1, 0, pairs_u=pairs)
            assert torch.equal(z0, z1) and torch.equal(v0, v1)
            words = ops._scheduling_words(dev)
            assert words.tolist() == [0, 0]
    # a sample of edges against the oracle
    sel = torch.arange(0, p.E, 997)
    sub_z, sub_v = ks.real_enc_fwd(p.a, p.rpos[sel], p.b.trans_vec, p.b.batch,
                                   p.edges[:, sel], 16, p.dist_max, 1.0, p.W, p.rvlen, -3.5, 1, 0)
    assert_close(z1.cpu()[sel], sub_z, "z sample")
    assert_close(v1.cpu()[sel], sub_v, "v sample")


@pytest.mark.parametrize("share", [0.6875, 0.25, 1.0 / 512])
def test_real_enc_fwd_launch_share_changes_no_bit(dev, share):
    """A launch that takes part of the GPU (fewer work-groups, more rounds each) gives the same
    bits, with the fixed stride and with the shared-counter scheduling; the share is restored."""
    for sizes, K, D in (([40, 3, 64, 17], 64, 16), ([256, 256], 16, 8)):
        p = Problem(sizes, H=8, K=K, D=D, seed=43)
        a, rpos, tv, bt, ed, W, rv = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.W, p.rvlen)
        for cutoff in (0.0, -3.5):
            z0, v0 = ops.real_enc_fwd(a, rpos, tv, bt, ed, K, p.dist_max, 1.0, W, rv, cutoff, 1, 0)
            with ops.launch_share(share):
                z1, v1 = ops.real_enc_fwd(a, rpos, tv, bt, ed, K, p.dist_max, 1.0, W, rv, cutoff, 1, 0)
            assert torch.equal(z0, z1) and torch.equal(v0, v1)
            assert ops._scheduling_words(dev).tolist() == [0, 0]
    from crystalformer_amd import lib
    assert lib.load().cf_get_launch_share() == 1.0


@pytest.mark.parametrize("N,C", [(1774, 128), (1774, 512), (5, 3), (100, 384), (0, 7)])
def test_column_sum(dev, N, C):
    g = torch.randn(N, C, generator=torch.Generator().manual_seed(N + C))
    out = ops.column_sum(g.to(dev))
    ref = g.double().sum(0).float()
    if N == 0:
        assert torch.equal(out.cpu(), torch.zeros(C))
    else:
        assert_close(out, ref, "column sums", rtol=2e-6)


def test_linear_function_gradients(dev):
    from crystalformer_amd.hip_funcs import LinearRowsHIP
    linear = LinearRowsHIP.apply
    g = torch.Generator().manual_seed(12)
    x, w, b = torch.randn(70, 32, generator=g), torch.randn(48, 32, generator=g), torch.randn(48, generator=g)
    go = torch.randn(70, 48, generator=g)
    xr, wr, br = (t.clone().requires_grad_() for t in (x, w, b))
    torch.nn.functional.linear(xr, wr, br).backward(go)
    xd, wd, bd = (t.to(dev).requires_grad_() for t in (x, w, b))
    y = linear(xd, wd, bd)
    y.backward(go.to(dev))
    assert_close(y.detach(), torch.nn.functional.linear(x, w, b), "y")
    for name, got, ref in (("gx", xd.grad, xr.grad), ("gw", wd.grad, wr.grad), ("gb", bd.grad, br.grad)):
        assert_close(got, ref, name, rtol=5e-6)


@pytest.mark.parametrize("N,C,K", [(1774, 128, 128), (1774, 512, 128), (1774, 128, 512), (70, 48, 32), (3, 5, 7),
                                   (600, 33, 100)])
def test_linear_weight_grad(dev, N, C, K):
    gen = torch.Generator().manual_seed(N + C + K)
    g, x = torch.randn(N, C, generator=gen), torch.randn(N, K, generator=gen)
    out = ops.linear_weight_grad(g.to(dev), x.to(dev))
    assert_close(out, (g.double().T @ x.double()).float(), "gW", rtol=3e-6)
    both, gb = ops.linear_weight_grad(g.to(dev), x.to(dev), with_bias=True)   # bias gradient from the same pass
    assert torch.equal(both, out)
    assert_close(gb, g.double().sum(0).float(), "gb", rtol=3e-6)


@pytest.mark.parametrize("clip", [1.0, 0.0, 1e4])
def test_fused_adamw_follows_torch(dev, clip):
    """clip + AdamW + inverse square-root schedule in one device-side update against
    torch.nn.utils.clip_grad_norm_ + torch.optim.AdamW + LambdaLR (the reference's training
    step, models/regression.py:106-135, :254-269) on 70 tensors of ragged sizes (more than
    one kernel-argument group of 64, chunks with tails, a single-element tensor)."""
    from crystalformer_amd.training import FusedAdamW, make_optimizer
    gen = torch.Generator().manual_seed(11)
    sizes = [1, 7, 128, 2048, 2049, 5000, 128 * 128, 512 * 128] + [100 + 37 * k for k in range(62)]

    class Bag(torch.nn.Module):
        def __init__(self):
            super().__init__()
            for k, n in enumerate(sizes):                 # odd ones named bias: no weight decay
                name = f"bias_{k}" if k % 2 else f"weight_{k}"
                self.register_parameter(name, torch.nn.Parameter(torch.randn(n, generator=gen)))

    ref, mine = Bag().to(dev), Bag().to(dev)
    mine.load_state_dict(ref.state_dict())
    opt, sch = make_optimizer(ref, lr=5e-4, weight_decay=1e-2, sch_decay=3.0)
    fused = FusedAdamW(mine, lr=5e-4, weight_decay=1e-2, sch_decay=3.0, clip_norm=clip)
    for step in range(6):
        scale = 10.0 ** (step - 3)                        # clip active on some steps only
        grads = [torch.randn(n, generator=gen) * scale for n in sizes]
        for p, q, g in zip(ref.parameters(), mine.parameters(), grads):
            p.grad, q.grad = g.to(dev), g.to(dev).clone()
        total = float(torch.linalg.vector_norm(torch.cat(grads).double()))
        if clip > 0:
            torch.nn.utils.clip_grad_norm_(ref.parameters(), clip)
        lr_ref = sch.get_last_lr()[0]
        opt.step()
        sch.step()
        fused.step()
        st = fused.state.cpu()
        assert float(st[0]) == step + 1
        assert abs(float(st[1]) - total) <= 1e-5 * total
        assert abs(float(st[2]) - lr_ref) <= 1e-6 * lr_ref
        for (name, p), q in zip(ref.named_parameters(), mine.parameters()):
            assert_close(q.detach(), p.detach(), f"{name} step {step}", rtol=2e-6)
    with pytest.raises(Exception):
        next(iter(mine.parameters())).grad = None
        fused.step()


@pytest.mark.parametrize("B,T", [(128, 1), (1, 1), (1000, 3), (257, 2)])
def test_l1_mean_loss_and_its_gradient(dev, B, T):
    """Loss and gradient of one launch against the reference's loss (restated in the oracle) and
    autograd; exact ties get a zero gradient, like torch's sign."""
    from oracle import torch_path as tp
    gen = torch.Generator().manual_seed(17)
    pred = torch.randn(B, T, generator=gen)
    target = torch.randn(B, T, generator=gen)
    target[::7] = pred[::7]                                   # ties
    ref_in = pred.clone().requires_grad_()
    ref = tp.l1_training_loss(ref_in, target)
    (ref * 3.0).backward()
    loss, grad = ops.l1_mean_loss(pred.to(dev), target.to(dev))
    ref_value = float(ref.detach())
    assert abs(float(loss) - ref_value) <= 2e-6 * abs(ref_value) + 1e-12
    assert torch.equal(grad.cpu() * 3.0, ref_in.grad) or float((grad.cpu() * 3.0 - ref_in.grad).abs().max()) < 1e-9
    mine_in = pred.to(dev).requires_grad_()
    out = hip_funcs.L1MeanLossHIP.apply(mine_in, target.to(dev))
    assert out.dim() == 0
    (out * 3.0).backward()
    assert float((mine_in.grad.cpu() - ref_in.grad).abs().max()) < 1e-9
    loss_only, none = ops.l1_mean_loss(pred.to(dev), target.to(dev), with_grad=False)
    assert none is None and float(loss_only) == float(loss)


@pytest.mark.parametrize("func", ["elu", "abs", "exp"])
@pytest.mark.parametrize("N,H,D,scaled", [(1774, 8, 16, True), (301, 3, 20, False), (5, 1, 4, True),
                                          (700, 16, 8, True),
                                          (40, 2, 6, True), (33, 3, 19, False)])   # widths off the 16-byte path
def test_gauss_exponents_bwd_kernel(dev, func, N, H, D, scaled):
    """Backward kernel against float64 autograd of a = coef * rho((alpha + shift) * scale),
    q_scaled = q * q_scale, with (scale, shift) constants; several blocks, ragged tails,
    head counts that do not divide the block and widths beyond one 16-column pass."""
    gen = torch.Generator().manual_seed(N + H + D)
    q = torch.randn(N, H, D, generator=gen)
    w = torch.randn(H, D, generator=gen) * 0.3
    ga = torch.randn(N, H, generator=gen)
    gqs = torch.randn(N, H, D, generator=gen) if scaled else None
    beta, lb, coef, q_scale = 0.1, 0.5, -0.37, 0.25
    used = torch.tensor([1.7, -0.2]) if scaled else None            # (scale, shift) of a normalising forward
    qd, wd = q.double().requires_grad_(), w.double().requires_grad_()
    alpha = (qd * wd[None]).sum(-1)
    alpha_n = (alpha + used[1].double()) * used[0].double() if used is not None else alpha
    if func == "elu":
        rho = (1 - lb) * torch.nn.functional.elu(alpha_n * (beta / (1 - lb))) + 1.0
    elif func == "abs":
        rho = (1 - lb) * alpha_n.abs() + lb
    else:
        rho = (1 - lb) * torch.exp(alpha_n * (beta / (1 - lb))) + lb
    obj = (rho * coef * ga.double()).sum()
    if scaled:
        obj = obj + (qd * q_scale * gqs.double()).sum()
    obj.backward()
    gq, gw = ops.gauss_exponents_bwd(ga.to(dev), gqs.to(dev) if scaled else None, q.to(dev), w.to(dev),
                                     alpha_n.detach().float().to(dev), used.to(dev) if scaled else None,
                                     func, beta, lb, coef, q_scale)
    assert_close(gq, qd.grad.float(), "gq")
    assert_close(gw, wd.grad.float(), "gw", rtol=3e-6)
    only_w = ops.gauss_exponents_bwd(ga.to(dev), None, q.to(dev), w.to(dev), alpha_n.detach().float().to(dev),
                                     used.to(dev) if scaled else None, func, beta, lb, coef, q_scale, want_gq=False)
    assert only_w[0] is None and torch.equal(only_w[1], gw)


def test_linear_weight_grad_grouped_equals_single_calls(dev):
    """Thirty-eight layers of ragged shapes (two kernel-argument groups of 32, with and without bias,
    different row counts and slice counts) in one grouped call: bit-identical to one call each."""
    gen = torch.Generator().manual_seed(21)
    shapes = [(1774, 128, 128), (1774, 512, 128), (1774, 128, 512), (70, 48, 32), (3, 5, 7), (600, 33, 100)]
    shapes = shapes * 6 + [(1774, 128, 128), (40, 16, 16)]
    layers, expect = [], []
    for k, (N, C, K) in enumerate(shapes):
        g, x = torch.randn(N, C, generator=gen).to(dev), torch.randn(N, K, generator=gen).to(dev)
        bias = k % 3 != 0
        expect.append(ops.linear_weight_grad(g, x, with_bias=True) if bias else (ops.linear_weight_grad(g, x), None))
        layers.append((g, x, torch.full((C, K), float("nan"), device=dev),
                       torch.full((C,), float("nan"), device=dev) if bias else None))
    ops.linear_weight_grad_grouped(layers)
    for k, ((g, x, gw, gb), (gw_ref, gb_ref)) in enumerate(zip(layers, expect)):
        assert torch.equal(gw, gw_ref), (k, shapes[k])
        assert (gb is None) == (gb_ref is None) and (gb is None or torch.equal(gb, gb_ref)), (k, shapes[k])


def test_deferred_weight_grads_match_immediate(dev):
    """Linear layers inside deferred_weight_grads(): parameter gradients appear at the
    context's exit and equal, bit for bit, those of the same backward pass without deferral."""
    from crystalformer_amd import hip_funcs
    gen = torch.Generator().manual_seed(5)
    x0 = torch.randn(300, 64, generator=gen).to(dev)
    target = torch.randn(300, 32, generator=gen).to(dev)

    def run(defer):
        torch.manual_seed(3)
        l1, l2 = torch.nn.Linear(64, 128).to(dev), torch.nn.Linear(128, 32, bias=False).to(dev)
        x = x0.clone().requires_grad_()
        h = torch.relu(hip_funcs.LinearRowsHIP.apply(x, l1.weight, l1.bias))
        loss = (hip_funcs.LinearRowsHIP.apply(h, l2.weight, None) - target).square().mean()
        if defer:
            with hip_funcs.deferred_weight_grads():
                loss.backward()
                assert l1.weight.grad is None and l2.weight.grad is None      # not yet
        else:
            loss.backward()
        return [x.grad, l1.weight.grad, l1.bias.grad, l2.weight.grad]

    for a, b in zip(run(True), run(False)):
        assert a is not None and torch.equal(a, b)
    assert hip_funcs._deferred is None


@pytest.mark.parametrize("defer", [False, True])
def test_fused_linear_function_grads(dev, defer):
    """FusedLinearHIP (three projections sharing an input and one bias vector; ReLU layer;
    residual layer) against float64 autograd of the same expression, immediate and deferred
    weight gradients."""
    from crystalformer_amd import hip_funcs
    gen = torch.Generator().manual_seed(17)
    N, K, C = 333, 64, 48
    x0 = torch.randn(N, K, generator=gen)
    ws = [torch.randn(C, K, generator=gen) * 0.2 for _ in range(3)]
    b3 = torch.randn(3 * C, generator=gen)
    w1, b1 = torch.randn(K, C, generator=gen) * 0.2, torch.randn(K, generator=gen)
    w2, b2 = torch.randn(K, K, generator=gen) * 0.2, torch.randn(K, generator=gen)
    tq, tk, tv = (torch.randn(N, C, generator=gen) for _ in range(3))

    def graph(x, ws, b3, w1, b1, w2, b2, lin3, lin_relu, lin_res):
        q, k, v = lin3(x, b3, ws)
        h = lin_relu(q * tq.to(q) + k * tk.to(q) - v * tv.to(q), b1, w1)        # (N, K)
        y = lin_res(h, b2, x, w2)                                                # + residual x
        return (y * y).mean()

    leaves64 = [t.double().requires_grad_() for t in (x0, *ws, b3, w1, b1, w2, b2)]
    x, a, b, c, bb, w1d, b1d, w2d, b2d = leaves64
    graph(x, (a, b, c), bb, w1d, b1d, w2d, b2d,
          lambda x, b3, ws: tuple(torch.nn.functional.linear(x, w, bs) for w, bs in zip(ws, b3.split(C))),
          lambda x, b, w: torch.relu(torch.nn.functional.linear(x, w, b)),
          lambda x, b, r, w: torch.nn.functional.linear(x, w, b) + r).backward()

    leaves = [t.to(dev).requires_grad_() for t in (x0, *ws, b3, w1, b1, w2, b2)]
    x, a, b, c, bb, w1d, b1d, w2d, b2d = leaves
    loss = graph(x, (a, b, c), bb, w1d, b1d, w2d, b2d,
                 lambda x, b3, ws: hip_funcs.FusedLinearHIP.apply(x, b3, None, False, False, *ws),
                 lambda x, b, w: hip_funcs.FusedLinearHIP.apply(x, b, None, True, False, w)[0],
                 lambda x, b, r, w: hip_funcs.FusedLinearHIP.apply(x, b, r, False, False, w)[0])
    if defer:
        with hip_funcs.deferred_weight_grads():
            loss.backward()
            assert a.grad is None and bb.grad is None
    else:
        loss.backward()
    names = ["x", "wq", "wk", "wv", "b3", "w1", "b1", "w2", "b2"]
    for name, t, r in zip(names, leaves, leaves64):
        assert t.grad is not None, name
        assert_close(t.grad, r.grad.float(), name, rtol=5e-6)


# ------------------------------------------------- reciprocal-space encoding
def _reci_problem(sizes, H, seed, a_lo=0.8, a_hi=4.0):
    b = make_sized_batch(sizes, seed)
    edges = tp.get_edge_index(b.sizes)
    g = torch.Generator().manual_seed(seed + 50)
    a = -(torch.rand(b.pos.shape[0], H, generator=g) * (a_hi - a_lo) + a_lo)
    rec, vcell = tp.reciprocal_vectors(b.trans_vec)
    rpos = tp.relative_positions(b.pos, edges)
    e_start = tp.edge_row_offsets(edges, b.pos.shape[0])
    return b, edges, a, rec, vcell, rpos, e_start, g


@pytest.mark.parametrize("sizes,H,R", [([1, 3, 5, 2], 4, 2), ([7, 1, 70, 12], 8, 2), ([4, 9], 2, 1), ([3, 130], 16, 3),
                                       ([5, 6], 3, 0)])
def test_reci_enc_fwd_bwd_against_oracle(dev, sizes, H, R):
    """Forward (z, S) and backward (ga) of the reciprocal-space kernels against the C restatement
    of the reference's kernels (double accumulation): rows longer than a wavefront, head counts
    that need padding, ranges 0..3.  z to 2e-5 absolute: the float phases reach tens of radians,
    so the sum itself carries ~1e-6 relative of its largest term."""
    b, edges, a, rec, vcell, rpos, e_start, g = _reci_problem(sizes, H, seed=H + R)
    kr = ops.kr_base(rpos.to(dev), rec.to(dev), b.batch.to(dev), edges.to(dev))
    kr_ref = tp.kr_base(b.pos, b.batch, b.trans_vec, edges)
    assert float((kr.cpu() - kr_ref).abs().max()) < 1e-5
    z_ref, se_ref = ks.reci_enc_fwd(a, kr_ref, rec, vcell, b.batch, edges, R)
    z, se = ops.reci_enc_fwd(a.to(dev), kr, rec.to(dev), vcell.to(dev), b.batch.to(dev), e_start.to(dev), R)
    assert_close(se, se_ref, "S", rtol=5e-6)
    assert float((z.cpu() - z_ref).abs().max()) < 2e-5
    gz = torch.randn(edges.shape[1], H, generator=g)
    ga_ref = ks.reci_enc_bwd(a, kr_ref, rec, b.batch, e_start, gz, se_ref, R)
    ga = ops.reci_enc_bwd(a.to(dev), kr, rec.to(dev), b.batch.to(dev), e_start.to(dev), gz.to(dev), se, R)
    assert_close(ga, ga_ref, "ga", rtol=1e-5)
    full_ref = ks.reci_enc_bwd(a, kr_ref, rec, b.batch, e_start, gz, se_ref, R, normalisation_grad=True)
    full = ops.reci_enc_bwd(a.to(dev), kr, rec.to(dev), b.batch.to(dev), e_start.to(dev), gz.to(dev), se, R,
                            normalisation_grad=True)
    assert_close(full, full_ref, "ga with the normalisation term", rtol=1e-5)


def test_reci_enc_clamp_and_function(dev):
    """Sums below 1e-6 (wide Gaussians): z takes log(1e-6) and the edge drops out of ga; the
    autograd Function returns the same z and ga and no other gradient."""
    from crystalformer_amd.hip_funcs import KernelManager, ReciPeriodicEncodingFuncCUDA
    b, edges, a, rec, vcell, rpos, e_start, g = _reci_problem([3, 4], 2, seed=9, a_lo=1e-4, a_hi=2e-3)
    kr_ref = tp.kr_base(b.pos, b.batch, b.trans_vec, edges)
    z_ref, se_ref = ks.reci_enc_fwd(a, kr_ref, rec, vcell, b.batch, edges, 2)
    assert bool((se_ref < 1e-6).any()) and bool((se_ref > 1e-3).any())
    old = KernelManager.LATTICE_RANGE
    KernelManager.LATTICE_RANGE = 2
    try:
        ad = a.to(dev).requires_grad_()
        z = ReciPeriodicEncodingFuncCUDA.apply(ad, kr_ref.to(dev), rec.to(dev), vcell.to(dev), b.batch.to(dev),
                                               edges.to(dev))
        gz = torch.randn(z.shape, generator=g)
        (z * gz.to(dev)).sum().backward()
    finally:
        KernelManager.LATTICE_RANGE = old
    solid = (se_ref - 1e-6).abs() > 1e-4                 # away from the switch itself
    assert float((z.detach().cpu() - z_ref)[solid].abs().max()) < 1e-4
    ga_ref = ks.reci_enc_bwd(a, kr_ref, rec, b.batch, e_start, gz, se_ref, 2)
    assert_close(ad.grad, ga_ref, "ga", rtol=2e-4)


@pytest.mark.parametrize("N,C,K,terms", [(1774, 128, 128, 3), (1774, 512, 128, 1), (1774, 128, 512, 1), (70, 64, 20, 2),
                                         (3, 64, 4, 1), (130, 192, 72, 3),
                                         (16500, 128, 128, 2)])                    # enough work-groups for full tiles
def test_linear_rows_nn(dev, N, C, K, terms):
    """Input-gradient kernel: mask(sum_i g_i W_i) + add against float64, with ragged row and
    column tails, one to three terms, with and without addend and mask."""
    gen = torch.Generator().manual_seed(N + C + K + terms)
    gs = [torch.randn(N, C, generator=gen) for _ in range(terms)]
    ws = [torch.randn(C, K, generator=gen) * 0.1 for _ in range(terms)]
    add, mask = torch.randn(N, K, generator=gen), torch.randn(N, K, generator=gen)
    base = sum(g.double() @ w.double() for g, w in zip(gs, ws))
    dg, dw = [g.to(dev) for g in gs], [w.to(dev) for w in ws]
    assert ops.linear_rows_nn_supported(dg[0], dw[0])
    assert_close(ops.linear_rows_nn(dg, dw), base.float(), "plain", rtol=3e-6)
    assert_close(ops.linear_rows_nn(dg, dw, add=add.to(dev)), (base + add.double()).float(), "add", rtol=3e-6)
    want = torch.where(mask.double() > 0, base, torch.zeros_like(base)) + add.double()
    assert_close(ops.linear_rows_nn(dg, dw, add=add.to(dev), mask=mask.to(dev)), want.float(), "mask + add", rtol=3e-6)
    assert not ops.linear_rows_nn_supported(torch.randn(4, 30, device=dev), torch.randn(30, 8, device=dev))


@pytest.mark.parametrize("defer", [False, True])
def test_fused_feed_forward_and_carried_input(dev, defer):
    """One block's dense path as the graphed training step runs it -- projections with the input
    carried to the residual of the output projection, then FusedFeedForwardHIP -- against float64
    autograd of the same expression: y = z + W2 relu(W1 z + b1) + b2, z = x + Wo (q * k + v) + bo."""
    from crystalformer_amd import hip_funcs
    gen = torch.Generator().manual_seed(29)
    N, E, F = 210, 64, 128
    shapes = dict(x=(N, E), wq=(E, E), wk=(E, E), wv=(E, E), b3=(3 * E,), wo=(E, E), bo=(E,), w1=(F, E), b1=(F,),
                  w2=(E, F), b2=(E,))
    vals = {k: torch.randn(*shp, generator=gen) * (0.2 if k.startswith("w") else 1.0) for k, shp in shapes.items()}
    t = torch.randn(N, E, generator=gen)
    lin = torch.nn.functional.linear
    r = {k: v.double().requires_grad_() for k, v in vals.items()}
    bq, bk, bv = r["b3"].split(E)
    z = r["x"] + lin(lin(r["x"], r["wq"], bq) * lin(r["x"], r["wk"], bk) + lin(r["x"], r["wv"], bv), r["wo"], r["bo"])
    y_ref = z + lin(torch.relu(lin(z, r["w1"], r["b1"])), r["w2"], r["b2"])
    (y_ref * t.double()).sum().backward()
    d = {k: v.to(dev).requires_grad_() for k, v in vals.items()}
    q, k, v, xc = hip_funcs.FusedLinearHIP.apply(d["x"], d["b3"], None, False, True, d["wq"], d["wk"], d["wv"])
    z, = hip_funcs.FusedLinearHIP.apply(q * k + v, d["bo"], xc, False, False, d["wo"])
    y = hip_funcs.FusedFeedForwardHIP.apply(z, d["w1"], d["b1"], d["w2"], d["b2"])
    assert_close(y, y_ref.detach().float(), "y", rtol=3e-6)
    if defer:
        with hip_funcs.deferred_weight_grads():
            (y * t.to(dev)).sum().backward()
            assert d["w1"].grad is None and d["b3"].grad is None
    else:
        (y * t.to(dev)).sum().backward()
    for name in shapes:
        assert d[name].grad is not None, name
        assert_close(d[name].grad, r[name].grad.float(), name, rtol=1e-5)


# ----------------------------------------- benchmark sizes at kernel level
def test_real_enc_bwd_pair_kernel_at_training_batch_size(dev):
    """The backward pair kernel at the training configuration's size (128 crystals, N = 1774,
    E = 56,440, H = 8, K = 64, D = 16, fixed cube): ga of a sample of atoms against the C
    oracle run on those atoms' edge rows, and gW through linearity -- with the incoming
    gradients zeroed outside the sampled rows the kernel's gW is the oracle's gW of the rows."""
    from crystalformer_amd.synthetic import make_config_batch
    b = make_config_batch("cfg4_train_b128")
    p = Problem(b, H=8, K=64, D=16, seed=71)
    p.a = p.a / (1.4 * 1.4) * 2.0
    gz, gv = p.randn(p.E, 8), p.randn(p.E, 8, 16)
    a, rpos, tv, bt, ed, W, es = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.W, p.e_start)
    pairs = ops.edge_pairs(p.b.sizes.to(dev))
    z, _ = ops.real_enc_fwd(a, rpos, tv, bt, ed, 64, p.dist_max, 1.0, W, None, 0.0, 2, 0, pairs_u=pairs)
    ga, gW = ops.real_enc_bwd(a, rpos, tv, bt, ed, es, z, gz.to(dev), gv.to(dev), 64, p.dist_max, 1.0, W, None,
                              0.0, 2, 0, pairs_u=pairs)
    atoms = torch.arange(5, p.N, 23)                                   # 77 atoms, crystals of every size
    in_rows = torch.zeros(p.N, dtype=torch.bool)
    in_rows[atoms] = True
    keep = in_rows[p.edges[0]]
    sub_edges = p.edges[:, keep].contiguous()
    sub_start = tp.edge_row_offsets(sub_edges, p.N)
    zc = z.cpu()
    ga_ref, gW_ref = ks.real_enc_bwd(p.a, p.rpos[keep], p.b.trans_vec, p.b.batch, sub_edges, sub_start, zc[keep],
                                     gz[keep], gv[keep], 64, p.dist_max, 1.0, p.W, None, 0.0, 2, 0)
    assert int(keep.sum()) > 2000
    ga_mag, gW_mag = ks.real_enc_bwd(p.a, p.rpos[keep], p.b.trans_vec, p.b.batch, sub_edges, sub_start, zc[keep],
                                     gz[keep], gv[keep], 64, p.dist_max, 1.0, p.W, None, 0.0, 2, 0, magnitude=True)
    assert_close(ga.cpu()[atoms], ga_ref[atoms], "ga", atol=RTOL * ga_mag[atoms].double())
    mask = keep.to(dev)
    _, gW_rows = ops.real_enc_bwd(a, rpos, tv, bt, ed, es, z, gz.to(dev) * mask[:, None],
                                  gv.to(dev) * mask[:, None, None], 64, p.dist_max, 1.0, W, None, 0.0, 2, 0,
                                  pairs_u=pairs)
    assert_close(gW_rows, gW_ref, "gW", atol=RTOL * gW_mag.double())
    assert float(gW.abs().max()) > 0 and torch.isfinite(gW).all()


def test_fused_dpa_at_stress_size(dev):
    """Attention forward and backward on the 16 cells of 200..444 atoms (E = 1.77 M edges, rows of
    up to 444 keys): every output against the C oracle, element by element."""
    from crystalformer_amd.synthetic import make_config_batch
    b = make_config_batch("cfg5_stress_b16")
    p = Problem(b, H=8, K=0, seed=72)
    q = p.randn(p.N, 8, 16) / 4.0
    k, v = p.randn(p.N, 8, 16), p.randn(p.N, 8, 16)
    a, bij = p.randn(p.E, 8) * 2, p.randn(p.E, 8, 16)
    out, prob = ops.fused_dpa_fwd(*to_dev(dev, q, k, v, a, bij, p.edges, p.e_start))
    out_ref, prob_ref = ks.fused_dpa_fwd(q, k, v, a, bij, p.edges, p.e_start)
    out_atol, bounds = dpa_atols(p, q, k, v, bij, prob_ref, out_ref)
    assert_close(out, out_ref, "out", atol=out_atol)
    assert_close(prob, prob_ref, "prob", atol=ATOL_PROB)
    go = p.randn(p.N, 8, 16)
    got = ops.fused_dpa_bwd(*to_dev(dev, q, k, v, bij, p.b.batch, p.edges, p.e_start, prob_ref, out_ref, go))
    ref = ks.fused_dpa_bwd(q, k, v, bij, p.edges, p.e_start, prob_ref, out_ref, go)
    atols = bounds(go)
    for name, x, y in zip(("gq", "gk", "gv", "gaij", "gbij"), got, ref):
        assert_close(x, y, name, atol=atols[name])


# ------------------------------------------- edge lists that are not dense blocks
def test_sparse_edge_list_takes_the_per_edge_kernels(dev):
    """An edge list sorted by source atom but with edges removed is not the dense per-crystal
    block layout: the encoding Functions notice on first sight and run the per-edge kernels
    (forward and backward against the C oracle on that very list), and the attention
    backward, which needs the blocks, raises instead of reading past the list."""
    p = Problem([3, 9, 1, 12], H=8, K=64, D=16, seed=73)
    gen = torch.Generator().manual_seed(4)
    keep = torch.rand(p.E, generator=gen) > 0.3
    edges = p.edges[:, keep].contiguous()
    rpos = p.rpos[keep].contiguous()
    e_start = tp.edge_row_offsets(edges, p.N)
    E = edges.shape[1]
    assert ops.dense_block_layout(p.b.batch.to(dev), edges.to(dev)) is None
    assert torch.equal(ops.dense_block_layout(p.b.batch.to(dev), p.edges.to(dev)).cpu(), p.b.sizes)
    assert ops.cached_edge_pairs(p.b.batch.to(dev), edges.to(dev), len(p.b.sizes)) is None
    hip_funcs.compile_kernels(2, 8, 16, 64, 16, False)
    a = p.a.to(dev).requires_grad_(True)
    W = p.W.to(dev).requires_grad_(True)
    bt, ed = p.b.batch.to(dev), edges.to(dev)
    z, v = hip_funcs.RealPeriodicEncodingWithProjFuncCUDA.apply(
        a, rpos.to(dev), None, p.b.trans_vec.to(dev), bt, ed, 64, p.dist_max, p.wscale, W)
    z_ref, v_ref = ks.real_enc_fwd(p.a, rpos, p.b.trans_vec, p.b.batch, edges, 64, p.dist_max, p.wscale, p.W,
                                   None, 0.0, 2, 0)
    assert_close(z, z_ref, "z")
    assert_close(v, v_ref, "v")
    gz, gv = p.randn(E, 8), p.randn(E, 8, 16)
    ((z * gz.to(dev)).sum() + (v * gv.to(dev)).sum()).backward()
    ga_ref, gW_ref = ks.real_enc_bwd(p.a, rpos, p.b.trans_vec, p.b.batch, edges, e_start, z_ref, gz, gv, 64,
                                     p.dist_max, p.wscale, p.W, None, 0.0, 2, 0)
    assert_close(a.grad, ga_ref, "ga")
    assert_close(W.grad, gW_ref.reshape(W.shape), "gW")
    q = (p.randn(p.N, 8, 16) / 4).to(dev).requires_grad_(True)
    k, val = p.randn(p.N, 8, 16).to(dev), p.randn(p.N, 8, 16).to(dev)
    out = hip_funcs.FusedDotProductAttentionCUDA.apply(q, k, val, z.detach(), v.detach(), bt, ed)
    out_ref, _ = ks.fused_dpa_fwd(q.detach().cpu(), k.cpu(), val.cpu(), z_ref, v_ref, edges, e_start)
    assert_close(out, out_ref, "out")
    with pytest.raises(lib.CrystalformerHipError, match="dense per-crystal edge blocks"):
        out.sum().backward()
    # an unsorted batch index is refused as well
    assert ops.dense_block_layout(torch.tensor([1, 0, 0], device=dev), tp.get_edge_index([1, 2]).to(dev)) is None


# ------------------------------------ lattice sums and attention in one launch
def test_fused_encoding_attention_on_the_simplified_model_batch(dev):
    """Blocks without Gaussian value bins: bias and attention from one launch against the CPU
    path's two steps (dense (E,R) lattice sum, per-crystal softmax) on the 32-crystal batch of the
    simplified configuration, and against the two separate kernels."""
    from crystalformer_amd.synthetic import make_config_batch
    b = make_config_batch("cfg1_simplified_b32")
    p = Problem(b, H=8, K=0, seed=91)
    p.a = -(1.0 + 0.1 * p.randn(p.N, 8)).clamp_min(0.5) / (2 * 1.4 * 1.4)
    q, k, v = p.randn(p.N, 8, 16), p.randn(p.N, 8, 16), p.randn(p.N, 8, 16)
    z_ref, _ = tp.periodic_encoding(p.a, p.b.pos, p.b.batch, p.b.trans_vec, p.edges, 2)
    out_ref, prob_ref = tp.indexed_attention(q.double(), k.double(), v.double(), p.b.sizes, p.edges, z_ref.double(),
                                             None)
    a, rpos, tv, bt, ed, es, qd, kd, vd = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start,
                                                 q / 4.0, k, v)
    out = ops.fused_enc_dpa_fwd(a, rpos, tv, bt, ed, es, qd, kd, vd, int(p.b.sizes.max()), None, 0.0, 2, 0)
    out_atol, _ = dpa_atols(p, q, k, v, None, prob_ref.float(), out_ref.float())
    assert_close(out, out_ref.float(), "out", atol=out_atol)
    z, _ = ops.real_enc_fwd(a, rpos, tv, bt, ed, 0, 1.0, 1.0, None, None, 0.0, 2, 0)
    two, _ = ops.fused_dpa_fwd(qd, kd, vd, z, None, ed, es)
    assert_close(out, two, "one launch vs two", rtol=2e-6)


@pytest.mark.parametrize("H,Dk,Dv,sizes", [(8, 16, 16, [1, 5, 70, 2]), (4, 8, 32, [3, 130]), (1, 5, 4, [7, 2]),
                                           (16, 16, 16, [9, 1]), (2, 64, 20, [4, 33])])
@pytest.mark.parametrize("cutoff,lr,mr", [(0.0, 2, 0), (-3.5, 2, 2), (-3.5, 1, 0), (4.0, 1, 1)])
def test_fused_encoding_attention_against_the_kernel_oracles(dev, H, Dk, Dv, sizes, cutoff, lr, mr):
    """Head counts and widths, rows longer than a wavefront, adaptive boxes per head, and an
    arbitrary sorted edge list with an atom that keeps no edge (its output row is zero)."""
    p = Problem(sizes, H=H, K=0, seed=92)
    g = p.g
    q = p.randn(p.N, H, Dk) / math.sqrt(Dk)
    k, v = p.randn(p.N, H, Dk), p.randn(p.N, H, Dv)
    keep = torch.rand(p.E, generator=g) > 0.25
    keep &= p.edges[0] != 3
    for edges, rpos in ((p.edges, p.rpos), (p.edges[:, keep].contiguous(), p.rpos[keep].contiguous())):
        e_start = tp.edge_row_offsets(edges, p.N)
        z_ref, _ = ks.real_enc_fwd(p.a, rpos, p.b.trans_vec, p.b.batch, edges, 0, 1.0, 1.0, None, p.rvlen, cutoff, lr,
                                   mr)
        out_ref, _ = ks.fused_dpa_fwd(q, k, v, z_ref, None, edges, e_start)
        max_row = int((e_start[1:] - e_start[:-1]).max())
        out = ops.fused_enc_dpa_fwd(*to_dev(dev, p.a, rpos, p.b.trans_vec, p.b.batch, edges, e_start, q, k, v),
                                    max_row, p.rvlen.to(dev), cutoff, lr, mr)
        assert_close(out, out_ref, "out")
        if edges.shape[1] < p.E and p.N > 3:
            assert float(out[3].abs().max()) == 0.0


def test_fused_encoding_attention_limits(dev):
    p = Problem([2, 3], H=8, K=0, seed=93)
    q = p.randn(p.N, 8, 16)
    args = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, q, q, q)
    with pytest.raises(lib.CrystalformerHipError, match="64 KB"):
        ops.fused_enc_dpa_fwd(*args, 4000)
    empty = ops.fused_enc_dpa_fwd(torch.zeros(0, 8, device=dev), torch.zeros(0, 3, device=dev),
                                  torch.zeros(0, 3, 3, device=dev), torch.zeros(0, dtype=torch.long, device=dev),
                                  torch.zeros(2, 0, dtype=torch.long, device=dev),
                                  torch.zeros(1, dtype=torch.long, device=dev), torch.zeros(0, 8, 16, device=dev),
                                  torch.zeros(0, 8, 16, device=dev), torch.zeros(0, 8, 16, device=dev), 0)
    assert empty.shape == (0, 8, 16)
    # the module takes the one-launch path only when nothing needs the bias afterwards
    assert hip_funcs.KernelManager.FUSE_ENCODING_ATTENTION
    a = p.a.to(dev).requires_grad_(True)
    hip_funcs.compile_kernels(2, 8, 16, 0, 16, False)
    got = hip_funcs.fused_encoding_attention(a, *args[1:5], *args[6:9])
    assert got is not None and not got.requires_grad


# ---- staged rings: the translations of every atom pair staged once, all blocks start from them

def _staged(dev, p, K, lr, weakest=None):
    rpos, tv = to_dev(dev, p.rpos, p.b.trans_vec)
    pairs = ops.edge_pairs(p.b.sizes.to(dev))
    weakest = float(p.a.max()) if weakest is None else weakest
    return rpos, tv, pairs, ops.staged_rings(rpos, tv, pairs, K, p.dist_max, p.wscale, lr, weakest)


@pytest.mark.parametrize("lr", [2, 1])
@pytest.mark.parametrize("H,K,D", [(8, 64, 16), (4, 16, 8), (1, 7, 3), (2, 100, 4), (16, 32, 8), (8, 64, 32),
                                   (8, 48, 20), (16, 128, 16)])
def test_real_enc_fwd_from_staged_rings(dev, H, K, D, lr):
    p = Problem([1, 3, 9, 2, 17, 1], H=H, K=K, D=D, seed=28)
    z_ref, v_ref = enc_fwd_ref(p, K, p.W, 0.0, lr, 0)
    rpos, tv, pairs, rings = _staged(dev, p, K, lr)
    assert rings is not None and rings.numel() * 4 == lib.load().cf_real_enc_ring_bytes(pairs.shape[0])
    a, ed, W = to_dev(dev, p.a, p.edges, p.W)
    z, v = ops.real_enc_fwd_rings(a, ed, pairs, rings, K, p.dist_max, p.wscale, W, lr)
    assert_close(z, z_ref, "z")
    assert_close(v, v_ref, "v", atol=v_atol(p, K, p.W, 0.0, lr, 0))
    # the same geometry again: the staged buffer is found, not rebuilt
    assert ops.staged_rings(rpos, tv, pairs, K, p.dist_max, p.wscale, lr, float(p.a.max())) is rings
    # a weaker bound on the exponents keeps more far translations: same result to the last bits
    _, _, _, rings0 = _staged(dev, p, K, lr, weakest=0.0)
    z0, v0 = ops.real_enc_fwd_rings(a, ed, pairs, rings0, K, p.dist_max, p.wscale, W, lr)
    assert rel_err(z0, z) < 1e-6 and rel_err(v0, v) < 1e-6


def test_staged_rings_serve_blocks_with_different_exponents(dev):
    """One staging, several exponent sets (the blocks of a model): each equals the pair kernel's result for its
    own exponents, on the pair kernel's own bits where no far translation is kept."""
    p = Problem([5, 11, 2, 30, 1], H=8, K=64, D=16, seed=33)
    exps = [p.a, p.a * 0.5, p.a * 3.0]
    rpos, tv, pairs, rings = _staged(dev, p, 64, 2, weakest=float(max(e.max() for e in exps)))
    bt, ed, W = to_dev(dev, p.b.batch, p.edges, p.W)
    for a_cpu in exps:
        a = a_cpu.to(dev)
        z0, v0 = ops.real_enc_fwd(a, rpos, tv, bt, ed, 64, p.dist_max, p.wscale, W, None, 0.0, 2, 0, pairs_u=pairs)
        z1, v1 = ops.real_enc_fwd_rings(a, ed, pairs, rings, 64, p.dist_max, p.wscale, W)
        assert rel_err(z1, z0) < 1e-6 and rel_err(v1, v0) < 1e-6
        p.a = a_cpu
        z_ref, v_ref = enc_fwd_ref(p, 64, p.W, 0.0, 2, 0)
        assert_close(z1, z_ref, "z")
        assert_close(v1, v_ref, "v", atol=v_atol(p, 64, p.W, 0.0, 2, 0))


@pytest.mark.parametrize("lr", [2, 1])
@pytest.mark.parametrize("H,K,D", [(8, 64, 16), (4, 16, 8), (16, 32, 16), (1, 7, 12)])
def test_real_enc_bwd_from_staged_rings(dev, H, K, D, lr):
    p = Problem([1, 3, 9, 2, 14, 1, 1, 1, 1, 20], H=H, K=K, D=D, seed=30)
    z_ref, v_ref = enc_fwd_ref(p, K, p.W, 0.0, lr, 0)
    gz, gv = p.randn(p.E, H), p.randn(*v_ref.shape)
    args = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv)
    _, _, pairs, rings = _staged(dev, p, K, lr)
    ga, gW = ops.real_enc_bwd(*args, K, p.dist_max, p.wscale, p.W.to(dev), None, 0.0, lr, 0, pairs_u=pairs,
                              rings=rings)
    ga_ref, gW_ref = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z_ref, gz, gv, K,
                                     p.dist_max, p.wscale, p.W, p.rvlen, 0.0, lr, 0)
    ga_atol, gW_atol = enc_bwd_atols(p, z_ref, gz, gv, K, p.W, 0.0, lr, 0)
    assert_close(ga, ga_ref, "ga", atol=ga_atol)
    assert_close(gW, gW_ref, "gW", atol=gW_atol)
    ga2, none = ops.real_enc_bwd(*args, K, p.dist_max, p.wscale, p.W.to(dev), None, 0.0, lr, 0, want_gW=False,
                                 pairs_u=pairs, rings=rings)
    assert none is None and torch.equal(ga2, ga)
    # only the value gradient, only the bias gradient
    for gz_, gv_ in ((None, args[8]), (args[7], None)):
        ga3, _ = ops.real_enc_bwd(*args[:7], gz_, gv_, K, p.dist_max, p.wscale, p.W.to(dev), None, 0.0, lr, 0,
                                  want_gW=False, pairs_u=pairs, rings=rings)
        ga4, _ = ops.real_enc_bwd(*args[:7], gz_, gv_, K, p.dist_max, p.wscale, p.W.to(dev), None, 0.0, lr, 0,
                                  want_gW=False, pairs_u=pairs)
        assert rel_err(ga3, ga4) < 1e-6


def test_staged_rings_limits(dev):
    p = Problem([3, 4], H=8, K=64, D=16, seed=34)
    assert _staged(dev, p, 64, 3)[3] is None                     # 343 translations: beyond the staged kernels
    assert _staged(dev, p, 0, 2)[3] is None                      # no value bins: nothing to stage for
    rpos, tv, pairs, rings = _staged(dev, p, 64, 2)
    a, ed, W = to_dev(dev, p.a, p.edges, p.W)
    with pytest.raises(lib.CrystalformerHipError, match="too small"):
        ops.real_enc_fwd_rings(a, ed, pairs, rings[:100], 64, p.dist_max, p.wscale, W)
    big = torch.zeros(8, 64, 64, device=dev)                     # D = 64: no staged kernel
    with pytest.raises(lib.CrystalformerHipError):
        ops.real_enc_fwd_rings(a, ed, pairs, rings, 64, p.dist_max, p.wscale, big)
    old = ops.STAGED_RINGS_MAX_BYTES
    ops.STAGED_RINGS_MAX_BYTES = 1000
    try:
        ops._ring_cache.clear()
        assert _staged(dev, p, 64, 2)[3] is None                 # too large to keep: blocks stage for themselves
    finally:
        ops.STAGED_RINGS_MAX_BYTES = old
    # backward: shapes its pair kernel does not take go to the other kernels, rings or not
    rpos, tv, pairs, rings = _staged(dev, p, 64, 2)
    z, v = ops.real_enc_fwd_rings(a, ed, pairs, rings, 64, p.dist_max, p.wscale, W)
    args = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start) + [z, torch.ones_like(z)]
    W32 = p.randn(8, 32, 64).to(dev)
    gv32 = p.randn(p.E, 8, 32).to(dev)
    with_rings = ops.real_enc_bwd(*args, gv32, 64, p.dist_max, p.wscale, W32, None, 0.0, 2, 0, pairs_u=pairs, rings=rings)
    without = ops.real_enc_bwd(*args, gv32, 64, p.dist_max, p.wscale, W32, None, 0.0, 2, 0, pairs_u=pairs)
    assert torch.equal(with_rings[0], without[0]) and torch.equal(with_rings[1], without[1])


@pytest.mark.parametrize("cutoff,lr,mr", [(-3.5, 2, 2), (-3.5, 1, 1), (-2.0, 2, 2), (5.0, 1, 1), (-3.5, 2, 0)])
@pytest.mark.parametrize("H,K,D", [(8, 64, 16), (4, 16, 8), (16, 32, 8), (2, 100, 4), (8, 64, 32)])
def test_real_enc_fwd_from_staged_rings_with_adaptive_boxes(dev, H, K, D, cutoff, lr, mr):
    """Adaptive boxes from staged rings: atom pairs whose half-widths all come out as lattice_range start from
    the rings, the others are staged by the pair kernel, each kind in a launch over its own list of units (16
    heads: all by the pair kernel).  Against the oracle and against the pair kernel alone; the problems hold
    pairs of both kinds."""
    p = Problem([1, 3, 9, 2, 17, 1, 6], H=H, K=K, D=D, seed=41)
    z_ref, v_ref = enc_fwd_ref(p, K, p.W, cutoff, lr, mr)
    rpos, tv, pairs, rings = _staged(dev, p, K, lr)
    a, bt, ed, W, rv = to_dev(dev, p.a, p.b.batch, p.edges, p.W, p.rvlen)
    z, v = ops.real_enc_fwd_rings(a, ed, pairs, rings, K, p.dist_max, p.wscale, W, lr, rpos, tv, bt, rv, cutoff, mr)
    assert_close(z, z_ref, "z")
    assert_close(v, v_ref, "v", atol=v_atol(p, K, p.W, cutoff, lr, mr))
    z1, v1 = ops.real_enc_fwd(a, rpos, tv, bt, ed, K, p.dist_max, p.wscale, W, rv, cutoff, lr, mr, pairs_u=pairs)
    assert rel_err(z, z1) < 1e-6 and rel_err(v, v1) < 1e-6
    # how the pairs split (the rule's integers are bit-exact on the device)
    R = ops.translation_ranges(a, rv, bt, cutoff, lr, mr)
    at_floor = (R == lr).all(-1).all(-1)
    both = at_floor[pairs[:, 2]] & at_floor[pairs[:, 3]]
    print("pairs from the rings:", int(both.sum()), "of", both.numel())


def test_adaptive_boxes_split_covers_both_kinds(dev):
    """The problems of the test above do hold atom pairs of both kinds for the default rule."""
    p = Problem([1, 3, 9, 2, 17, 1, 6], H=8, K=64, D=16, seed=41)
    a, bt, rv = to_dev(dev, p.a, p.b.batch, p.rvlen)
    pairs = ops.edge_pairs(p.b.sizes.to(dev))
    R = ops.translation_ranges(a, rv, bt, -3.5, 2, 2)
    at_floor = (R == 2).all(-1).all(-1)
    both = at_floor[pairs[:, 2]] & at_floor[pairs[:, 3]]
    assert 0 < int(both.sum()) < both.numel()
