"""Pins for the reciprocal-space part of the oracle (CPU only): the kernel-level C restatement
and the torch-path restatement against the full-cube sum in float64, against each other (they
enumerate the half space differently), against the Poisson summation identity with the
real-space lattice sum, and the backward against float64 autograd of the sum."""
import itertools
import math

import pytest
import torch

from oracle import kernel_semantics as ks
from oracle import torch_path as tp
from tests.helpers import make_sized_batch, rel_err


def problem(sizes, H=4, seed=0, a_lo=0.05, a_hi=1.5):
    b = make_sized_batch(sizes, seed)
    edges = tp.get_edge_index(b.sizes)
    g = torch.Generator().manual_seed(seed + 50)
    a = -(torch.rand(b.pos.shape[0], H, generator=g) * (a_hi - a_lo) + a_lo)
    rec, vcell = tp.reciprocal_vectors(b.trans_vec)
    kr = tp.kr_base(b.pos, b.batch, b.trans_vec, edges)
    return b, edges, a, rec, vcell, kr


def full_cube_sum(b, edges, a, R, weight_k2=False):
    """sum over n in [-R,R]^3 of (k^2)? exp(a k^2) cos(k.r), float64, (E,H)."""
    rec, _ = tp.reciprocal_vectors(b.trans_vec.double())
    grid = torch.tensor(list(itertools.product(range(-R, R + 1), repeat=3)), dtype=torch.float64)
    k = grid @ rec                                                  # (B,T,3)
    k2 = (k * k).sum(-1)                                            # (B,T)
    rel = (b.pos.double()[edges[1]] - b.pos.double()[edges[0]])
    be = b.batch[edges[0]]
    phase = (k[be] * rel[:, None, :]).sum(-1)                       # (E,T)
    w = torch.exp(a[edges[0]][:, :, None] * k2[be][:, None, :])     # (E,H,T)
    if weight_k2:
        w = w * k2[be][:, None, :]
    return (w * torch.cos(phase)[:, None, :]).sum(-1)


@pytest.mark.parametrize("R", [1, 2, 3])
def test_forward_equals_full_cube_sum(R):
    # exponents of the size the model produces (a = -rho * scale_reci^2 / 2, scale_reci = 2.2, rho >= 0.5)
    b, edges, a, rec, vcell, kr = problem([1, 3, 5, 2], seed=R, a_lo=0.8, a_hi=4.0)
    S = full_cube_sum(b, edges, a.double(), R)
    assert float(S.min()) > 1e-3                                    # well away from the clamp here
    z_ref = torch.log(S) + (1.5 * torch.log(-4 * math.pi * a.double()) -
                            torch.log(vcell.double())[b.batch, None])[edges[0]]
    z, se = ks.reci_enc_fwd(a, kr, rec, vcell, b.batch, edges, R)
    assert rel_err(se, S.float()) < 2e-6
    assert float((z - z_ref.float()).abs().max()) < 2e-5
    cos_kr, k2, vc = tp.reciprocal_half_terms(b.pos, b.batch, b.trans_vec, edges, R)
    assert cos_kr.shape[1] == ((2 * R + 1) ** 3 + 1) // 2
    z_tp = tp.reciprocal_bias(a, cos_kr, k2, vc, edges[0], b.batch)
    assert float((z_tp - z_ref.float()).abs().max()) < 5e-5        # float32 phases up to ~40 rad
    assert float((z_tp - z).abs().max()) < 5e-5


def test_poisson_summation_links_reciprocal_and_real_space():
    """(1/V)(2 pi s^2)^{3/2} sum_k exp(-s^2 k^2 / 2) cos(k.r) = sum_n exp(-|r + L n|^2 / (2 s^2)):
    the reciprocal-space z at a = -s^2/2 equals the real-space lattice-sum bias at
    a = -1/(2 s^2) once both ranges are wide enough."""
    b = make_sized_batch([2, 4, 1], seed=4)
    edges = tp.get_edge_index(b.sizes)
    rec, vcell = tp.reciprocal_vectors(b.trans_vec)
    kr = tp.kr_base(b.pos, b.batch, b.trans_vec, edges)
    N = b.pos.shape[0]
    sigma = torch.tensor([[1.1, 1.6, 2.2]]).expand(N, 3).contiguous()
    z_reci, _ = ks.reci_enc_fwd(-0.5 * sigma ** 2, kr, rec, vcell, b.batch, edges, 7)
    dist2 = tp.lattice_dist2(b.pos.double(), b.batch, b.trans_vec.double(), edges, 7)
    z_real = tp.lattice_logsumexp((-0.5 / sigma.double() ** 2)[edges[0]], dist2)
    assert float((z_reci - z_real.float()).abs().max()) < 3e-5


def test_clamp_of_small_and_negative_sums():
    """Wide Gaussians (a -> 0-) make the truncated sum oscillate through zero: below 1e-6 the
    logarithm is taken of 1e-6 and the backward contribution of the edge is zero."""
    b, edges, a, rec, vcell, kr = problem([3, 4], H=2, seed=9, a_lo=1e-4, a_hi=2e-3)
    S = full_cube_sum(b, edges, a.double(), 2)
    low = S < 1e-6
    assert bool(low.any()) and bool((~low).any())
    z, se = ks.reci_enc_fwd(a, kr, rec, vcell, b.batch, edges, 2)
    log_ci = (1.5 * torch.log(-4 * math.pi * a.double()) - torch.log(vcell.double())[b.batch, None])[edges[0]]
    want = torch.log(S.clamp(min=1e-6)) + log_ci
    solid = (S - 1e-6).abs() > 1e-3                                 # away from the switch itself
    assert float((z.double() - want)[solid].abs().max()) < 1e-4
    e_start = tp.edge_row_offsets(edges, b.pos.shape[0])
    gz = torch.ones_like(z)
    ga = ks.reci_enc_bwd(a, kr, rec, b.batch, e_start, gz, se, 2)
    dS = full_cube_sum(b, edges, a.double(), 2, weight_k2=True)
    contrib = torch.where(se.double() < 1e-6, torch.zeros_like(dS), dS / se.double())
    want_ga = torch.zeros_like(a, dtype=torch.float64).index_add_(0, edges[0], contrib)
    assert rel_err(ga, want_ga.float()) < 1e-4


def test_backward_is_the_gradient_of_log_sum_only():
    """ga = d/da sum_e gz log S (autograd on the float64 full-cube sum); the derivative 1.5/a of
    the normalisation term is absent, as in the reference's kernel
    (models/kernels/reci_enc_bwd.cu:41-69)."""
    b, edges, a, rec, vcell, kr = problem([2, 5, 3], seed=2, a_lo=0.8, a_hi=4.0)
    e_start = tp.edge_row_offsets(edges, b.pos.shape[0])
    g = torch.Generator().manual_seed(1)
    gz = torch.randn(edges.shape[1], a.shape[1], generator=g)
    ad = a.double().requires_grad_()
    S = full_cube_sum(b, edges, ad, 2)
    (torch.log(S) * gz.double()).sum().backward()
    _, se = ks.reci_enc_fwd(a, kr, rec, vcell, b.batch, edges, 2)
    ga = ks.reci_enc_bwd(a, kr, rec, b.batch, e_start, gz, se, 2)
    assert rel_err(ga, ad.grad.float()) < 5e-6
    # and it differs from the gradient of the full z by exactly 1.5 / a * (row sums of gz)
    full = ad.grad + 1.5 / a.double() * torch.zeros_like(a, dtype=torch.float64).index_add_(0, edges[0], gz.double())
    ad2 = a.double().requires_grad_()
    z_full = torch.log(full_cube_sum(b, edges, ad2, 2)) + (1.5 * torch.log(-4 * math.pi * ad2))[edges[0]]
    (z_full * gz.double()).sum().backward()
    assert rel_err(full.float(), ad2.grad.float()) < 1e-6
    ga_full = ks.reci_enc_bwd(a, kr, rec, b.batch, e_start, gz, se, 2, normalisation_grad=True)
    assert rel_err(ga_full, ad2.grad.float()) < 5e-6


def test_kr_base_is_the_phase_per_reciprocal_vector():
    b, edges, a, rec, vcell, kr = problem([3, 2], seed=5)
    for e in range(edges.shape[1]):
        i, j = int(edges[0, e]), int(edges[1, e])
        r = (b.pos[j] - b.pos[i]).double()
        want = rec[b.batch[i]].double() @ r
        assert float((kr[e].double() - want).abs().max()) < 1e-5
    # <b_d, t_c> = 2 pi delta_dc: a shift by a lattice vector changes the phase by 2 pi
    prod = rec.double() @ b.trans_vec.double().transpose(1, 2)
    assert float((prod - 2 * math.pi * torch.eye(3, dtype=torch.float64)).abs().max()) < 1e-4
