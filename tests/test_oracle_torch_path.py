"""Pins of the torch-path oracle (oracle/torch_path.py) that need no reference
import: brute force in float64, closed forms, library routines, invariants."""
import itertools
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import torch_path as tp
from tests.helpers import Problem, make_sized_batch, rel_err


# ------------------------------------------------------------------ integers
def brute_edges(sizes):
    src, dst, off = [], [], 0
    for n in sizes:
        for i in range(n):
            for j in range(n):
                src.append(off + i)
                dst.append(off + j)
        off += n
    return torch.tensor([src, dst], dtype=torch.long).reshape(2, -1)


@pytest.mark.parametrize("sizes", [[1], [3], [1, 2, 5], [4, 1, 1, 7], [2, 0, 3]])
def test_edge_index_bruteforce(sizes):
    e = tp.get_edge_index(sizes)
    assert e.dtype == torch.long and e.is_contiguous()
    assert torch.equal(e, brute_edges(sizes))
    assert e.shape[1] == sum(n * n for n in sizes)
    assert bool((e[0][1:] >= e[0][:-1]).all())


def test_edge_index_empty():
    assert tp.get_edge_index([]).shape == (2, 0)


def test_edge_index_accepts_tensor():
    assert torch.equal(tp.get_edge_index(torch.tensor([2, 3])), brute_edges([2, 3]))


def test_row_offsets_sizes_starts():
    sizes = [3, 1, 4]
    e = tp.get_edge_index(sizes)
    N = sum(sizes)
    start = tp.edge_row_offsets(e, N)
    expect = [0]
    for n in sizes:
        for _ in range(n):
            expect.append(expect[-1] + n)
    assert start.tolist() == expect
    batch = torch.tensor(sum([[b] * n for b, n in enumerate(sizes)], []))
    assert tp.crystal_sizes(batch).tolist() == sizes
    assert tp.crystal_sizes(batch, 5).tolist() == sizes + [0, 0]
    assert tp.crystal_starts(torch.tensor(sizes)).tolist() == [0, 3, 4, 8]


# ------------------------------------------------------------------ geometry
@pytest.mark.parametrize("r", [0, 1, 2])
def test_translation_grid_order(r):
    g = tp.translation_grid(r)
    expect = list(itertools.product(range(-r, r + 1), repeat=3))   # first index slowest
    assert g.shape == ((2 * r + 1) ** 3, 3)
    assert g.tolist() == [list(map(float, t)) for t in expect]


def test_det_and_reciprocal():
    b = make_sized_batch([1, 1, 1, 1], seed=5)
    t = b.trans_vec.double()
    assert torch.allclose(tp.det_3x3(t), torch.linalg.det(t), rtol=1e-12, atol=0)
    rec, vol = tp.reciprocal_vectors(t)
    eye = torch.eye(3, dtype=torch.float64) * (2 * math.pi)
    assert torch.allclose(rec @ t.transpose(1, 2), eye.expand(4, 3, 3), atol=1e-9)
    assert torch.allclose(vol, torch.linalg.det(t))


def brute_dist2(pos, batch, trans, edges, r):
    pos, trans = pos.double(), trans.double()
    E = edges.shape[1]
    grid = list(itertools.product(range(-r, r + 1), repeat=3))
    out = torch.zeros(E, len(grid), dtype=torch.float64)
    for e in range(E):
        i, j = int(edges[0, e]), int(edges[1, e])
        L = trans[int(batch[i])]
        for k, (n1, n2, n3) in enumerate(grid):
            d = pos[j] - pos[i] + n1 * L[0] + n2 * L[1] + n3 * L[2]
            out[e, k] = (d * d).sum()
    return out


@pytest.mark.parametrize("r", [0, 1, 2])
def test_lattice_dist2_bruteforce(r):
    b = make_sized_batch([2, 3], seed=2)
    edges = tp.get_edge_index(b.sizes)
    got = tp.lattice_dist2(b.pos, b.batch, b.trans_vec, edges, r)
    ref = brute_dist2(b.pos, b.batch, b.trans_vec, edges, r)
    assert got.shape == ref.shape
    assert rel_err(got, ref) < 5e-7
    # slicing over edges does not change values
    part = tp.lattice_dist2(b.pos, b.batch, b.trans_vec, edges, r, 3, 9)
    assert torch.equal(part, got[3:9])


def test_lattice_dist2_r0_is_plain_distance():
    b = make_sized_batch([4], seed=3)
    edges = tp.get_edge_index(b.sizes)
    got = tp.lattice_dist2(b.pos.double(), b.batch, b.trans_vec.double(), edges, 0)[:, 0]
    d = b.pos.double()[edges[1]] - b.pos.double()[edges[0]]
    assert torch.allclose(got, (d * d).sum(-1), rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------- alpha pipeline
def test_positive_elu_unit_cases():
    x = torch.linspace(-50, 50, 101, dtype=torch.float64)
    rho = tp.positive_elu(x, 0.5, 0.1)
    assert float(tp.positive_elu(torch.zeros(1), 0.5, 0.1)) == 1.0
    assert bool((rho > 0.5).all())                       # lower bound is approached, never crossed
    assert abs(float(tp.positive_elu(torch.tensor(-1e4, dtype=torch.float64), 0.5, 0.1)) - 0.5) < 1e-9
    assert bool((rho[1:] > rho[:-1]).all())              # monotone
    # linear branch: slope beta for x > 0
    assert abs(float(rho[-1] - rho[-2]) - 0.1 * 1.0) < 1e-12


def test_gaussian_exponents_statistics_and_storage():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(50, 4, 8, generator=g, dtype=torch.float64)
    w = torch.randn(32, generator=g, dtype=torch.float64)
    scale = torch.zeros(2, dtype=torch.float64)
    a = tp.gaussian_exponents(q, w, scale, False, True, 0.5, 0.1, 1.4)
    assert a.shape == (50, 4) and bool((a < 0).all())
    assert float(scale.abs().sum()) == 0.0               # eval mode stores nothing
    # invert rho on the linear/elu branches to recover the normalised alpha
    rho = a / (-0.5 * 1.4 ** -2)
    alpha = torch.where(rho >= 1, (rho - 1) / 0.1, torch.log((rho - 1) / 0.5 + 1) * 0.5 / 0.1)
    assert abs(float(alpha.mean())) < 1e-9 and abs(float(alpha.std()) - 1) < 1e-9
    raw = torch.einsum("nhd,hd->nh", q, w.view(4, 8))
    assert torch.allclose(alpha, (raw - raw.mean()) / raw.std(), atol=1e-9)
    # training mode stores (1/std, -mean) once and then reuses it
    tp.gaussian_exponents(q, w, scale, True, True, 0.5, 0.1, 1.4)
    assert torch.allclose(scale, torch.stack([1 / raw.std(), -raw.mean()]))
    stored = scale.clone()
    a2 = tp.gaussian_exponents(q * 3 + 1, w, scale, True, True, 0.5, 0.1, 1.4)
    assert torch.equal(scale, stored)
    raw2 = torch.einsum("nhd,hd->nh", q * 3 + 1, w.view(4, 8))
    expect = tp.positive_elu((raw2 + stored[1]) * stored[0], 0.5, 0.1) * (-0.5 / 1.4 ** 2)
    assert torch.allclose(a2, expect)
    # without normalisation: alpha = 0 -> a = -1/(2 r0^2)
    a0 = tp.gaussian_exponents(torch.zeros(3, 4, 8), w.float(), torch.zeros(2), False, False, 0.5, 0.1, 2.0)
    assert torch.allclose(a0, torch.full((3, 4), -1.0 / 8.0))


# -------------------------------------------------------------- lattice sum
def test_logsumexp_orthorhombic_factorises():
    """For an orthorhombic cell the cube sum is a product of three 1-D sums."""
    L = torch.tensor([3.0, 4.5, 6.0], dtype=torch.float64)
    trans = torch.diag(L)[None]
    pos = torch.tensor([[0.3, 0.2, 0.1], [1.7, 3.9, 2.5]], dtype=torch.float64)
    batch = torch.zeros(2, dtype=torch.long)
    edges = tp.get_edge_index([2])
    r = 2
    a = torch.tensor([[-0.3, -1.1], [-0.05, -2.0]], dtype=torch.float64)
    d2 = tp.lattice_dist2(pos, batch, trans, edges, r)
    z = tp.lattice_logsumexp(a[edges[0]], d2)
    for e in range(4):
        i, j = int(edges[0, e]), int(edges[1, e])
        x = pos[j] - pos[i]
        for h in range(2):
            prod = 1.0
            for d in range(3):
                prod *= sum(math.exp(float(a[i, h]) * float(x[d] + n * L[d]) ** 2) for n in range(-r, r + 1))
            assert abs(float(z[e, h]) - math.log(prod)) < 1e-10


def test_logsumexp_limits():
    p = Problem([3, 2], H=2, K=0, seed=4)
    d2 = tp.lattice_dist2(p.b.pos.double(), p.b.batch, p.b.trans_vec.double(), p.edges, 2)
    a = torch.full((p.E, 2), -200.0, dtype=torch.float64)
    off = d2.min(dim=1).values > 1e-9                      # self edges have d2min = 0 with multiplicity 1
    z = tp.lattice_logsumexp(a, d2)
    # sharply peaked: z -> a * d2min (up to the log of the multiplicity of the minimum, here 1)
    assert torch.allclose(z[off], (a * d2.min(dim=1, keepdim=True).values)[off], atol=1e-6)
    # r = 0: a single term
    d0 = tp.lattice_dist2(p.b.pos.double(), p.b.batch, p.b.trans_vec.double(), p.edges, 0)
    a = p.a.double()[p.edges[0]]
    assert torch.allclose(tp.lattice_logsumexp(a, d0), a * d0, atol=1e-12)
    # library routine on brute-force distances
    ref = torch.logsumexp(brute_dist2(p.b.pos, p.b.batch, p.b.trans_vec, p.edges, 1)[:, None, :] * a[:, :, None], -1)
    got = tp.lattice_logsumexp(a, tp.lattice_dist2(p.b.pos.double(), p.b.batch, p.b.trans_vec.double(), p.edges, 1))
    assert torch.allclose(got, ref, atol=1e-9)


def test_dist2_multiset_symmetry():
    """(i,j) and (j,i) see the same multiset of distances on a symmetric cube,
    hence equal bias for equal exponents."""
    p = Problem([4], H=1, K=0, seed=6)
    d2 = tp.lattice_dist2(p.b.pos.double(), p.b.batch, p.b.trans_vec.double(), p.edges, 2)
    a = torch.full((p.E, 1), -0.37, dtype=torch.float64)
    z = tp.lattice_logsumexp(a, d2).view(4, 4)
    assert torch.allclose(z, z.t(), atol=1e-10)


# ---------------------------------------------------------- Gaussian basis
def test_gaussian_basis_shape_peak_width():
    m, K, ws = 14.0, 64, 1.0
    mu = m / K
    centers = torch.arange(1, K + 1, dtype=torch.float64) * mu
    g = tp.gaussian_basis((centers ** 2)[None], m, K, ws)[0]          # distance = every centre in turn
    assert g.shape == (K, K)
    assert torch.allclose(torch.diagonal(g), torch.ones(K, dtype=torch.float64))     # peak 1 at own centre
    assert torch.allclose(g, g.t())                                                    # uniform spacing
    # one bin away = one standard deviation (sigma = ws * mu): exp(-1/2)
    assert torch.allclose(torch.diagonal(g, 1), torch.full((K - 1,), math.exp(-0.5), dtype=torch.float64))
    assert torch.allclose(torch.diagonal(g, 3), torch.full((K - 3,), math.exp(-4.5), dtype=torch.float64))
    # width scale stretches sigma
    g2 = tp.gaussian_basis((centers ** 2)[None], m, K, 2.0)[0]
    assert torch.allclose(torch.diagonal(g2, 2), torch.full((K - 2,), math.exp(-0.5), dtype=torch.float64))
    # first centre is at mu, not 0
    g0 = tp.gaussian_basis(torch.zeros(1, 1, dtype=torch.float64), m, K, ws)[0, 0]
    assert abs(float(g0[0]) - math.exp(-0.5)) < 1e-12


def brute_value_average(a_e, d2, m, K, ws):
    E, H = a_e.shape
    R = d2.shape[1]
    out = torch.zeros(E, H, K, dtype=torch.float64)
    for e in range(E):
        for h in range(H):
            w = [math.exp(float(a_e[e, h]) * float(d2[e, r])) for r in range(R)]
            tot = sum(w)
            for k in range(K):
                c = (k + 1) * m / K
                sig = ws * m / K
                out[e, h, k] = sum(w[r] / tot * math.exp(-((c - math.sqrt(float(d2[e, r]))) ** 2) / (2 * sig * sig))
                                   for r in range(R))
    return out


def test_gaussian_value_average_bruteforce_and_special_cases():
    p = Problem([2, 1], H=2, K=6, D=3, seed=8)
    d2 = tp.lattice_dist2(p.b.pos.double(), p.b.batch, p.b.trans_vec.double(), p.edges, 1)
    a_e = p.a.double()[p.edges[0]]
    got = tp.gaussian_value_average(a_e, d2, 7.0, 6, 1.3)
    assert torch.allclose(got, brute_value_average(a_e, d2, 7.0, 6, 1.3), atol=1e-12)
    # r = 0: the average is the basis at the plain distance
    d0 = tp.lattice_dist2(p.b.pos.double(), p.b.batch, p.b.trans_vec.double(), p.edges, 0)
    s0 = tp.gaussian_value_average(a_e, d0, 7.0, 6, 1.0)
    assert torch.allclose(s0, tp.gaussian_basis(d0, 7.0, 6, 1.0).expand(-1, 2, -1), atol=1e-12)
    # all translations at the same distance: weights drop out
    same = torch.full((3, 5), 2.25, dtype=torch.float64)
    s = tp.gaussian_value_average(torch.tensor([[-0.1, -3.0]] * 3, dtype=torch.float64), same, 7.0, 6, 1.0)
    assert torch.allclose(s, tp.gaussian_basis(same[:, :1], 7.0, 6, 1.0).expand(-1, 2, -1), atol=1e-12)


def test_project_value_pe_matches_einsum():
    g = torch.Generator().manual_seed(1)
    s = torch.randn(5, 3, 7, generator=g, dtype=torch.float64)
    W3 = torch.randn(3, 4, 7, generator=g, dtype=torch.float64)
    WE = torch.randn(5, 3, 4, 7, generator=g, dtype=torch.float64)
    assert torch.allclose(tp.project_value_pe(s, W3), torch.einsum("ehk,hdk->ehd", s, W3))
    assert torch.allclose(tp.project_value_pe(s, W3[None]), torch.einsum("ehk,hdk->ehd", s, W3))
    assert torch.allclose(tp.project_value_pe(s, WE), torch.einsum("ehk,ehdk->ehd", s, WE))


def test_periodic_encoding_chunking_invariant():
    p = Problem([3, 1, 4], H=4, K=8, D=5, seed=9)
    args = (p.a, p.b.pos, p.b.batch, p.b.trans_vec, p.edges, 1, 8, 9.0, 1.0, p.W)
    z1, v1 = tp.periodic_encoding(*args)
    z2, v2 = tp.periodic_encoding(*args, chunk_elems=300)
    assert torch.equal(z1, z2) and torch.equal(v1, v2)
    z3, v3 = tp.periodic_encoding(p.a, p.b.pos, p.b.batch, p.b.trans_vec, p.edges, 1, 0)
    assert v3 is None and torch.equal(z3, z1)
    WE = p.randn(p.E, 4, 5, 8)
    _, v4 = tp.periodic_encoding(p.a, p.b.pos, p.b.batch, p.b.trans_vec, p.edges, 1, 8, 9.0, 1.0, WE, chunk_elems=300)
    _, s = tp.periodic_encoding(p.a, p.b.pos, p.b.batch, p.b.trans_vec, p.edges, 1, 8, 9.0, 1.0, None)
    assert torch.allclose(v4, torch.einsum("ehk,ehdk->ehd", s, WE), atol=1e-6)


# ---------------------------------------------------------------- attention
def test_indexed_attention_single_crystal_is_sdpa():
    g = torch.Generator().manual_seed(2)
    n, H, D = 6, 3, 8
    q, k, v = (torch.randn(n, H, D, generator=g, dtype=torch.float64) for _ in range(3))
    edges = tp.get_edge_index([n])
    out, prob = tp.indexed_attention(q, k, v, [n], edges, None, None)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1)).transpose(0, 1)
    assert torch.allclose(out, ref, atol=1e-12)
    assert torch.allclose(prob.view(n, n, H).sum(1), torch.ones(n, H, dtype=torch.float64))


def test_indexed_attention_multi_crystal_bias_values():
    g = torch.Generator().manual_seed(3)
    sizes = [2, 4, 1]
    N, H, D = sum(sizes), 2, 4
    q, k, v = (torch.randn(N, H, D, generator=g, dtype=torch.float64) for _ in range(3))
    edges = tp.get_edge_index(sizes)
    E = edges.shape[1]
    bias = torch.randn(E, H, generator=g, dtype=torch.float64)
    vals = torch.randn(E, H, D, generator=g, dtype=torch.float64)
    out, prob = tp.indexed_attention(q, k, v, sizes, edges, bias, vals)
    # dense block-diagonal restatement
    logits = torch.full((N, N, H), -float("inf"), dtype=torch.float64)
    logits[edges[0], edges[1]] = torch.einsum("ehd,ehd->eh", q[edges[0]], k[edges[1]]) / math.sqrt(D) + bias
    P = torch.softmax(logits, dim=1)
    dense_vals = torch.zeros(N, N, H, D, dtype=torch.float64)
    dense_vals[edges[0], edges[1]] = vals
    ref = torch.einsum("ijh,ijhd->ihd", P, v[None] + dense_vals)
    assert torch.allclose(out, ref, atol=1e-12)
    assert torch.allclose(prob, P[edges[0], edges[1]], atol=1e-12)


def test_avr_pool_is_segment_mean():
    x = torch.arange(24, dtype=torch.float64).view(8, 3)
    got = tp.avr_pool(x, [3, 1, 4])
    ref = torch.stack([x[0:3].mean(0), x[3:4].mean(0), x[4:8].mean(0)])
    assert torch.equal(got, ref)
