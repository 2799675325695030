"""Pins of the kernel-semantics oracle (oracle/kernels_ref.c): agreement with
the independently written torch-path oracle under the fixed cube, autograd /
finite differences for the backward passes, brute force and geometric
invariants for the adaptive translation boxes."""
import itertools
import math

import pytest
import torch

from oracle import kernel_semantics as ks
from oracle import torch_path as tp
from tests.helpers import Problem, rel_err


@pytest.fixture(scope="module", autouse=True)
def _built():
    ks.build()


@pytest.mark.parametrize("K,proj", [(0, False), (12, False), (12, True), (64, True)])
def test_fwd_matches_torch_path_under_fixed_cube(K, proj):
    p = Problem([3, 1, 5], H=4, K=K, D=6, seed=11)
    W = p.W if proj else None
    z, v = ks.real_enc_fwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, K, p.dist_max, p.wscale, W,
                           None, 0.0, 2, 0)
    z_ref, v_ref = tp.periodic_encoding(p.a.double(), p.b.pos.double(), p.b.batch, p.b.trans_vec.double(),
                                        p.edges, 2, K, p.dist_max, p.wscale, None if W is None else W.double())
    assert rel_err(z, z_ref) < 2e-6
    if K > 0:
        assert rel_err(v, v_ref) < 2e-6
    else:
        assert v is None


def test_fwd_per_edge_and_per_atom_projection():
    for mode in ("edge", "atom"):
        p = Problem([2, 3], H=2, K=5, D=3, seed=12, W_mode=mode)
        _, s = ks.real_enc_fwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, 5, 9.0, 1.0, None, None, 0.0, 1, 0)
        _, v = ks.real_enc_fwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, 5, 9.0, 1.0, p.W, None, 0.0, 1, 0)
        Wsel = p.W if mode == "edge" else p.W[p.edges[0]]
        assert rel_err(v, torch.einsum("ehk,ehdk->ehd", s, Wsel)) < 1e-6


def test_bwd_matches_autograd_of_torch_path():
    p = Problem([3, 2, 4], H=4, K=10, D=5, seed=13)
    a = p.a.double().requires_grad_(True)
    W = p.W.double().requires_grad_(True)
    z, v = tp.periodic_encoding(a, p.b.pos.double(), p.b.batch, p.b.trans_vec.double(), p.edges, 2, 10,
                                p.dist_max, p.wscale, W)
    gz, gv = p.randn(*z.shape), p.randn(*v.shape)
    ((z * gz).sum() + (v * gv).sum()).backward()
    ga, gW = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z.detach().float(),
                             gz, gv, 10, p.dist_max, p.wscale, p.W, None, 0.0, 2, 0)
    assert rel_err(ga, a.grad) < 5e-6
    assert rel_err(gW, W.grad) < 5e-6
    # without projection, and bias-only
    a2 = p.a.double().requires_grad_(True)
    z2, s2 = tp.periodic_encoding(a2, p.b.pos.double(), p.b.batch, p.b.trans_vec.double(), p.edges, 2, 10,
                                  p.dist_max, p.wscale, None)
    gs = p.randn(*s2.shape)
    ((z2 * gz).sum() + (s2 * gs).sum()).backward()
    ga2, none = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z2.detach().float(),
                                gz, gs, 10, p.dist_max, p.wscale, None, None, 0.0, 2, 0)
    assert none is None and rel_err(ga2, a2.grad) < 5e-6
    a3 = p.a.double().requires_grad_(True)
    z3, _ = tp.periodic_encoding(a3, p.b.pos.double(), p.b.batch, p.b.trans_vec.double(), p.edges, 2, 0)
    (z3 * gz).sum().backward()
    ga3, _ = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z3.detach().float(),
                             gz, None, 0, 1.0, 1.0, None, None, 0.0, 2, 0)
    assert rel_err(ga3, a3.grad) < 5e-6


def test_bwd_finite_differences_adaptive_box():
    """Central differences through the C forward itself, with adaptive boxes
    (the box of a head does not change under a 1e-3 relative step here)."""
    p = Problem([2, 3], H=2, K=6, D=4, seed=14)
    cut, lr, mr = 2.0, 1, 1     # fixed positive radius: boxes independent of a
    def fwd(a):
        return ks.real_enc_fwd(a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, 6, 9.0, 1.0, p.W, p.rvlen, cut, lr, mr)
    z, v = fwd(p.a)
    gz, gv = p.randn(*z.shape), p.randn(*v.shape)
    ga, gW = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z, gz, gv, 6, 9.0, 1.0,
                             p.W, p.rvlen, cut, lr, mr)
    loss = lambda zz, vv: float((zz.double() * gz).sum() + (vv.double() * gv).sum())
    for (i, h) in [(0, 0), (2, 1), (4, 0)]:
        eps = 2e-3
        ap, am = p.a.clone(), p.a.clone()
        ap[i, h] += eps
        am[i, h] -= eps
        fd = (loss(*fwd(ap)) - loss(*fwd(am))) / (2 * eps)
        assert abs(fd - float(ga[i, h])) < 2e-2 * max(1.0, abs(fd)), (fd, float(ga[i, h]))


def brute_ranges(a, rvl, cutoff, lr, mr):
    a32 = torch.tensor(a, dtype=torch.float32)
    c = torch.tensor(cutoff, dtype=torch.float32)
    if cutoff == 0:
        return [lr] * 3
    if cutoff < 0:
        c = torch.sqrt(torch.tensor(-0.5, dtype=torch.float32) / a32) * (-c)
    out = []
    for d in range(3):
        num = (c + torch.tensor(0.01, dtype=torch.float32)) * torch.tensor(rvl[d], dtype=torch.float32)
        pi_f = float(torch.tensor(3.141592654, dtype=torch.float32))
        R = math.ceil(float(num) / (2.0 * pi_f))
        out.append(max(R, mr) if mr > 0 else R)
    return out


@pytest.mark.parametrize("cutoff,lr,mr", [(0.0, 2, 0), (-3.5, 2, 2), (-3.5, 2, 0), (4.0, 1, 0), (-1.0, 3, 1)])
def test_translation_ranges_rule(cutoff, lr, mr):
    p = Problem([2, 3, 1], H=4, K=0, seed=15)
    R = ks.translation_ranges(p.a, p.rvlen, p.b.batch, cutoff, lr, mr)
    assert R.dtype == torch.int32 and R.shape == (p.N, 4, 3)
    for i in range(p.N):
        for h in range(4):
            assert R[i, h].tolist() == brute_ranges(float(p.a[i, h]), p.rvlen[p.b.batch[i]].tolist(), cutoff, lr, mr)
    if cutoff == 0.0:
        assert bool((R == lr).all())
    if mr > 0:
        assert bool((R >= mr).all())


def test_translation_box_contains_cutoff_sphere():
    """Geometric invariant of the rule: every lattice point within the cut-off
    radius lies inside the box [-R_d, R_d]^3."""
    p = Problem([1, 1, 1, 1], H=2, K=0, seed=16)
    cutoff = 7.0
    R = ks.translation_ranges(p.a, p.rvlen, p.b.batch, cutoff, 0, 0)
    for b in range(4):
        L = p.b.trans_vec[b].double()
        Rb = R[b, 0].tolist()
        big = [r + 3 for r in Rb]
        for n in itertools.product(*[range(-x, x + 1) for x in big]):
            vec = n[0] * L[0] + n[1] * L[1] + n[2] * L[2]
            if float(vec.norm()) <= cutoff:
                assert all(abs(n[d]) <= Rb[d] for d in range(3)), (n, Rb)


def test_fwd_adaptive_box_bruteforce():
    p = Problem([2, 2], H=2, K=4, D=3, seed=17)
    cut, lr, mr = -2.0, 1, 0
    z, s = ks.real_enc_fwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, 4, 6.0, 1.0, None, p.rvlen, cut, lr, mr)
    R = ks.translation_ranges(p.a, p.rvlen, p.b.batch, cut, lr, mr)
    assert len({tuple(r.tolist()) for r in R.view(-1, 3)}) > 1      # boxes really differ
    for e in range(p.E):
        i = int(p.edges[0, e])
        L = p.b.trans_vec[p.b.batch[i]].double()
        for h in range(2):
            r1, r2, r3 = R[i, h].tolist()
            a = float(p.a[i, h])
            d2 = []
            for n in itertools.product(range(-r1, r1 + 1), range(-r2, r2 + 1), range(-r3, r3 + 1)):
                vec = p.rpos[e].double() + n[0] * L[0] + n[1] * L[1] + n[2] * L[2]
                d2.append(float((vec * vec).sum()))
            w = [math.exp(a * x) for x in d2]
            assert abs(float(z[e, h]) - math.log(sum(w))) < 2e-5
            for k in range(4):
                c = (k + 1) * 6.0 / 4
                ref = sum(wi * math.exp(-((c - math.sqrt(x)) ** 2) / (2 * (6.0 / 4) ** 2)) for wi, x in zip(w, d2)) / sum(w)
                assert abs(float(s[e, h, k]) - ref) < 2e-6


def test_fused_dpa_matches_torch_path_and_autograd():
    p = Problem([3, 1, 4], H=2, K=0, seed=18)
    Dk = 4
    q, k, v = (p.randn(p.N, 2, Dk).double().requires_grad_(True) for _ in range(3))
    bias = p.randn(p.E, 2).double().requires_grad_(True)
    vals = p.randn(p.E, 2, Dk).double().requires_grad_(True)
    out, prob = tp.indexed_attention(q, k, v, p.b.sizes, p.edges, bias, vals)
    go = p.randn(*out.shape).double()
    (out * go).sum().backward()
    qs = (q / math.sqrt(Dk)).detach()
    out_c, prob_c = ks.fused_dpa_fwd(qs, k, v, bias, vals, p.edges, p.e_start)
    assert rel_err(out_c, out) < 1e-6 and rel_err(prob_c, prob) < 1e-6
    gq, gk, gv, ga, gb = ks.fused_dpa_bwd(qs, k, v, vals, p.edges, p.e_start, prob_c, out_c, go)
    assert rel_err(gq, q.grad * math.sqrt(Dk)) < 2e-6      # gradient wrt the pre-scaled query
    assert rel_err(gk, k.grad) < 2e-6 and rel_err(gv, v.grad) < 2e-6
    assert rel_err(ga, bias.grad) < 2e-6 and rel_err(gb, vals.grad) < 2e-6
    # softmax Jacobian property: the logit gradients of one query sum to zero
    row_sum = torch.zeros(p.N, 2, dtype=torch.float64).index_add_(0, p.edges[0], ga.double())
    assert float(row_sum.abs().max()) < 1e-5
    # without bias / values
    out2, _ = ks.fused_dpa_fwd(qs, k, v, None, None, p.edges, p.e_start)
    ref2, _ = tp.indexed_attention(q.detach(), k.detach(), v.detach(), p.b.sizes, p.edges, None, None)
    assert rel_err(out2, ref2) < 1e-6


def test_irregular_mean_and_minimum_distance():
    p = Problem([3, 1, 6], H=1, K=0, seed=19)
    x = p.randn(p.N, 7)
    start = tp.crystal_starts(p.b.sizes)
    assert rel_err(ks.irregular_mean(x, start), tp.avr_pool(x.double(), p.b.sizes)) < 1e-6
    d2 = tp.lattice_dist2(p.b.pos.double(), p.b.batch, p.b.trans_vec.double(), p.edges, 2)
    got = ks.minimum_distance(p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.rvlen, 0.0, 2, 0)
    assert rel_err(got, d2.min(dim=1).values) < 1e-5
    # a positive cut-off picks the box from the rule; it then contains the true nearest image
    got2 = ks.minimum_distance(p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.rvlen, 9.0, 0, 0)
    d2big = tp.lattice_dist2(p.b.pos.double(), p.b.batch, p.b.trans_vec.double(), p.edges, 4)
    assert rel_err(got2, d2big.min(dim=1).values) < 1e-5


# ---- the tolerance helpers (not restatements of reference code, but the element-wise parity bounds of
# the GPU tests are built from them, so they are pinned like everything else)
def _dense_translations(p, lattice_range):
    """(E,T) squared distances of every edge over the fixed cube, float64, meshgrid-'ij' order."""
    r = range(-lattice_range, lattice_range + 1)
    n = torch.tensor(list(itertools.product(r, r, r)), dtype=torch.float64)          # (T,3)
    shift = n @ p.b.trans_vec.double()[p.b.batch[p.edges[0]]]                         # (E,T,3)
    return ((p.rpos.double()[:, None, :] + shift) ** 2).sum(-1)


def test_conditioning_helper_is_the_sum_of_absolute_sensitivities():
    """ref_real_enc_fwd_cond against central finite differences in float64: s_k = sum_n w_n g_k(d_n) / S
    with every translation's distance (inside g) and squared distance (inside w) perturbed on its own;
    cond is the sum over translations of |ds/d ln d_n| + |ds/d ln d2_n| (S held fixed).  A missing
    factor, a wrong width or a signed instead of absolute sum fails this."""
    p = Problem([2, 3], H=2, K=8, D=4, seed=31)
    lr, K, dist_max, ws = 1, 8, 9.0, 0.8
    cond = ks.real_enc_fwd_cond(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, K, dist_max, ws, None, 0.0, lr, 0)
    d2 = _dense_translations(p, lr)                                                   # (E,T)
    a = p.a.double()[p.edges[0]]                                                      # (E,H)
    mu = dist_max / K
    centres = torch.arange(1, K + 1, dtype=torch.float64) * mu

    def parts(dd, dd2):
        """unnormalised weights (E,H,T) from dd2 and Gaussians (E,T,K) from dd"""
        w = torch.exp(a[:, :, None] * (dd2[:, None, :] - d2.min(dim=1).values[:, None, None]))
        g = torch.exp(-((centres[None, None, :] - dd[:, :, None]) / (math.sqrt(2.0) * ws * mu)) ** 2)
        return w, g
    d = d2.sqrt()
    w0, g0 = parts(d, d2)
    S = w0.sum(-1)                                                                    # (E,H), held fixed
    T = d2.shape[1]
    expect = torch.zeros(p.E, 2, K, dtype=torch.float64)
    h = 1e-6
    for n in range(T):
        bump = torch.zeros(T, dtype=torch.float64)
        bump[n] = h
        # relative perturbation of the distance inside the Gaussians
        _, gp = parts(d * (1 + bump), d2)
        _, gm = parts(d * (1 - bump), d2)
        ds_dist = torch.einsum("eht,etk->ehk", w0, gp - gm) / (2 * h) / S[:, :, None]
        # relative perturbation of the squared distance inside the weights
        wp, _ = parts(d, d2 * (1 + bump))
        wm, _ = parts(d, d2 * (1 - bump))
        ds_w = torch.einsum("eht,etk->ehk", wp - wm, g0) / (2 * h) / S[:, :, None]
        expect += ds_dist.abs() + ds_w.abs()
    assert rel_err(cond, expect) < 1e-5
    assert float((cond.double() - expect).abs().max()) <= 1e-5 * float(expect.abs().max())
    # and it really bounds a float32 evaluation's error to first order: recompute s from distances
    # rounded to float32 and compare with the float64 s
    s64 = torch.einsum("eht,etk->ehk", w0, g0) / S[:, :, None]
    w32, g32 = parts(d2.float().sqrt().double(), d2.float().double())
    s32 = torch.einsum("eht,etk->ehk", w32, g32) / S[:, :, None]
    assert bool(((s32 - s64).abs() <= 2.0 ** -23 * expect + 1e-15).all())


def test_backward_magnitude_helper_is_the_sum_of_absolute_terms():
    """ref_real_enc_bwd_magnitude against a brute-force expansion in float64: every individual product
    that enters ga (gz p d2; p d2 g W gv; -(p d2)(p g W gv)) and gW (p g gv) is formed as its own
    tensor entry and the absolute values are summed."""
    p = Problem([2, 3], H=2, K=6, D=3, seed=32)
    lr, K = 1, 6
    z, _ = ks.real_enc_fwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, K, 9.0, 1.0, p.W, None, 0.0, lr, 0)
    gz, gv = p.randn(p.E, 2), p.randn(p.E, 2, 3)
    ga_mag, gW_mag = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z, gz, gv, K, 9.0,
                                     1.0, p.W, None, 0.0, lr, 0, magnitude=True)
    d2 = _dense_translations(p, lr)                                                   # (E,T)
    a = p.a.double()[p.edges[0]]
    logit = a[:, :, None] * d2[:, None, :]
    prob = torch.softmax(logit, dim=-1)                                               # (E,H,T)
    mu = 9.0 / K
    centres = torch.arange(1, K + 1, dtype=torch.float64) * mu
    g = torch.exp(-((centres[None, None, :] - d2.sqrt()[:, :, None]) / (math.sqrt(2.0) * mu)) ** 2)   # (E,T,K)
    W = p.W.double()[0]                                                               # (H,D,K)
    gv64, gz64 = gv.double(), gz.double()
    t1 = gz64[:, :, None] * prob * d2[:, None, :]                                     # (E,H,T)
    t2 = torch.einsum("eht,et,etk,hdk,ehd->ehtkd", prob, d2, g, W, gv64)
    pd2 = prob * d2[:, None, :]
    t3 = -torch.einsum("ehm,eht,etk,hdk,ehd->ehmtkd", pd2, prob, g, W, gv64)
    per_edge = t1.abs().sum(-1) + t2.abs().sum((-1, -2, -3)) + t3.abs().sum((-1, -2, -3, -4))
    ga_expect = torch.zeros(p.N, 2, dtype=torch.float64).index_add_(0, p.edges[0], per_edge)
    gW_terms = torch.einsum("eht,etk,ehd->ehtdk", prob, g, gv64)
    gW_expect = gW_terms.abs().sum((0, 2))[None]                                      # (1,H,D,K)
    assert rel_err(ga_mag, ga_expect) < 1e-5 and rel_err(gW_mag, gW_expect) < 1e-5
    # the signed sums are the gradients themselves, and never exceed the magnitudes
    ga, gW = ks.real_enc_bwd(p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, z, gz, gv, K, 9.0, 1.0,
                             p.W, None, 0.0, lr, 0)
    signed = torch.zeros(p.N, 2, dtype=torch.float64).index_add_(
        0, p.edges[0], t1.sum(-1) + t2.sum((-1, -2, -3)) + t3.sum((-1, -2, -3, -4)))
    assert rel_err(ga, signed) < 1e-5 and rel_err(gW, gW_terms.sum((0, 2))[None]) < 1e-5
    assert bool((ga.abs() <= ga_mag * (1 + 1e-6)).all()) and bool((gW.abs() <= gW_mag * (1 + 1e-6)).all())
