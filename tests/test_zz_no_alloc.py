"""The backward of the periodic encoding through the entry point that brings its own scratch
(``cf_real_enc_bwd_static``): same gradients, bit for bit, as ``cf_real_enc_bwd`` with a
caller-provided workspace, on two calls in a row, the second one smaller (the shared scratch
then still holds the first call's partial results)."""
import pytest
import torch

from crystalformer_amd import lib, ops
from crystalformer_amd.lib import ptr, stream_handle
from tests.helpers import Problem, to_dev

pytestmark = pytest.mark.gpu


def bwd_static(dev, p, z, gz, gv, W, rvlen, cutoff, lr, mr, pairs, want_gW=True):
    """ctypes call of cf_real_enc_bwd_static; only the outputs are allocated (by the caller)."""
    L = lib.load()
    a, rpos, tv, bt, ed, es = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start)
    N, H = a.shape
    E, B = ed.shape[1], tv.shape[0]
    K = 0 if W is None else W.shape[-1]
    D = 0 if W is None else W.shape[-2]
    W_num = 0 if W is None else (1 if W.dim() == 3 else W.shape[0])
    ga = torch.full_like(a, float("nan"))
    gW = torch.full_like(W, float("nan")) if (want_gW and W is not None) else None
    rc = L.cf_real_enc_bwd_static(ptr(a), ptr(rpos), ptr(tv), ptr(bt), ptr(ed), ptr(es), ptr(z), ptr(gz), ptr(gv),
                                  N, H, E, B, K, D, float(p.dist_max), float(p.wscale), ptr(W), W_num, ptr(rvlen),
                                  float(cutoff), lr, mr, ptr(pairs), 0 if pairs is None else pairs.shape[0],
                                  ptr(ga), ptr(gW), stream_handle(dev))
    return rc, ga, gW


@pytest.mark.parametrize("use_pairs", [True, False])
def test_static_scratch_backward_matches_the_workspace_entry_point(dev, use_pairs):
    L = lib.load()
    assert L.cf_static_scratch_bytes() == 32 << 20
    first = Problem([20, 7, 33, 1, 12, 40], H=8, K=64, D=16, seed=81)
    second = Problem([3, 9, 2], H=8, K=64, D=16, seed=82)              # smaller: stale scratch beyond its extent
    for p in (first, second, first):
        for cutoff, lr, mr in ((0.0, 2, 0), (-3.5, 2, 2)):
            a, rpos, tv, bt, ed, es, W, rv = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges,
                                                    p.e_start, p.W, p.rvlen)
            pairs = ops.edge_pairs(p.b.sizes.to(dev)) if use_pairs else None
            z, _ = ops.real_enc_fwd(a, rpos, tv, bt, ed, 64, p.dist_max, p.wscale, W, rv, cutoff, lr, mr,
                                    pairs_u=pairs)
            gz, gv = p.randn(p.E, 8).to(dev), p.randn(p.E, 8, 16).to(dev)
            ga_ref, gW_ref = ops.real_enc_bwd(a, rpos, tv, bt, ed, es, z, gz, gv, 64, p.dist_max, p.wscale, W, rv,
                                              cutoff, lr, mr, pairs_u=pairs)
            rc, ga, gW = bwd_static(dev, p, z, gz, gv, W, rv, cutoff, lr, mr, pairs)
            assert rc == 0, L.cf_last_error()
            torch.cuda.synchronize()
            assert torch.equal(ga, ga_ref) and torch.equal(gW, gW_ref)
            # bias-only gradient (no value gradient): gW is cleared, ga still exact
            ga_ref2, _ = ops.real_enc_bwd(a, rpos, tv, bt, ed, es, z, gz, None, 64, p.dist_max, p.wscale, W, rv,
                                          cutoff, lr, mr, pairs_u=pairs)
            rc, ga2, gW2 = bwd_static(dev, p, z, gz, None, W, rv, cutoff, lr, mr, pairs)
            assert rc == 0 and torch.equal(ga2, ga_ref2) and float(gW2.abs().max()) == 0.0


def test_static_scratch_backward_rejects_what_does_not_fit(dev):
    """Sizes whose scratch exceeds the built-in 32 MiB are refused before anything is launched."""
    L = lib.load()
    N, H, E, K, D = 6000, 8, 2_000_000, 64, 16
    assert L.cf_real_enc_bwd_workspace(N, H, E, K, D, 1, 1) > L.cf_static_scratch_bytes()
    rc = L.cf_real_enc_bwd_static(0, 0, 0, 0, 0, 0, 0, 0, 0, N, H, E, 16, K, D, 14.0, 1.0, 0, 1, 0, 0.0, 2, 0, 0, 0,
                                  0, 0, 0)
    assert rc != 0
    msg = L.cf_last_error().decode()
    assert "built-in buffer holds 33554432" in msg and "cf_real_enc_bwd with a workspace" in msg


def test_static_scratch_backward_allocates_nothing_and_runs_under_capture(dev):
    """What the entry point is for.  (1) A warmed call with preallocated outputs leaves the device's
    free memory and torch's allocator untouched.  (2) The same call recorded into a HIP graph (where
    hipMalloc is not allowed) and replayed several times, with eager work and synchronisations in
    between, gives the eager result bit for bit every time."""
    L = lib.load()
    p = Problem([20, 7, 33, 1, 12], H=8, K=64, D=16, seed=83)
    a, rpos, tv, bt, ed, es, W = to_dev(dev, p.a, p.rpos, p.b.trans_vec, p.b.batch, p.edges, p.e_start, p.W)
    pairs = ops.edge_pairs(p.b.sizes.to(dev))
    z, _ = ops.real_enc_fwd(a, rpos, tv, bt, ed, 64, p.dist_max, p.wscale, W, pairs_u=pairs)
    gz, gv = p.randn(p.E, 8).to(dev), p.randn(p.E, 8, 16).to(dev)
    ga_ref, gW_ref = ops.real_enc_bwd(a, rpos, tv, bt, ed, es, z, gz, gv, 64, p.dist_max, p.wscale, W, pairs_u=pairs)
    ga, gW = torch.empty_like(a), torch.empty_like(W)
    N, H = a.shape
    E, B = ed.shape[1], tv.shape[0]

    def call(stream):
        return L.cf_real_enc_bwd_static(ptr(a), ptr(rpos), ptr(tv), ptr(bt), ptr(ed), ptr(es), ptr(z), ptr(gz),
                                        ptr(gv), N, H, E, B, 64, 16, float(p.dist_max), float(p.wscale), ptr(W), 1,
                                        0, 0.0, 2, 0, ptr(pairs), pairs.shape[0], ptr(ga), ptr(gW), stream)
    assert call(stream_handle(dev)) == 0, L.cf_last_error()           # warm: module loaded, symbol looked up
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    reserved_before, allocated_before = torch.cuda.memory_reserved(), torch.cuda.memory_allocated()
    ga.fill_(float("nan"))
    gW.fill_(float("nan"))
    assert call(stream_handle(dev)) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert (torch.cuda.memory_reserved(), torch.cuda.memory_allocated()) == (reserved_before, allocated_before)
    assert torch.equal(ga, ga_ref) and torch.equal(gW, gW_ref)
    # under stream capture
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = call(stream_handle(dev))
    assert rc == 0, L.cf_last_error()
    for rep in range(3):
        ga.fill_(float("nan"))
        gW.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(ga, ga_ref) and torch.equal(gW, gW_ref), rep
        again, _ = ops.real_enc_bwd(a, rpos, tv, bt, ed, es, z, gz, gv, 64, p.dist_max, p.wscale, W, pairs_u=pairs)
        assert torch.equal(again, ga_ref)                             # eager work between replays
        torch.cuda.synchronize()
