"""Host build of the arithmetic the device kernels share with no one else -- the translation half-width
rule with its clamps, and the index arithmetic of the dense per-crystal edge blocks
(crystalformer_amd/csrc/cf_index_rules.h) -- compiled with g++ and checked on the CPU: against the C
oracle and the torch-path oracle value by value, on the inputs a kernel must survive (exponents that are
zero, positive, infinite, NaN; reciprocal lengths that are zero), and under AddressSanitizer + UBSan
together with the C oracle itself (tests/host/san_driver.c)."""
import ctypes
import math
import os
import subprocess

import pytest
import torch

from oracle import kernel_semantics as ks
from oracle import torch_path as tp

HOST = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host")


@pytest.fixture(scope="module")
def host():
    subprocess.check_call(["make", "-C", HOST, "-B", "libcf_host_rules.so"], stdout=subprocess.DEVNULL)
    return ctypes.CDLL(os.path.join(HOST, "libcf_host_rules.so"))


def host_ranges(host, a, rvlen, batch, cutoff, lattice_range, minimum_range):
    a, batch = a.contiguous().float(), batch.contiguous().long()
    rvlen = None if rvlen is None else rvlen.contiguous().float()
    N, H = a.shape
    out = torch.empty((N, H, 3), dtype=torch.int32)
    host.host_translation_ranges(ctypes.c_void_p(a.data_ptr()),
                                 ctypes.c_void_p(0 if rvlen is None else rvlen.data_ptr()),
                                 ctypes.c_void_p(batch.data_ptr()), ctypes.c_int64(N), ctypes.c_int64(H),
                                 ctypes.c_double(cutoff), ctypes.c_int(lattice_range), ctypes.c_int(minimum_range),
                                 ctypes.c_void_p(out.data_ptr()))
    return out


def test_range_rule_equals_the_oracle_for_finite_negative_exponents(host):
    """The kernels' rule (float quotient first, the double division only near whole numbers) gives the
    integers of the reference's rule (models/kernels/real_enc_fwd.cu:58-85, restated in the C oracle)
    for every finite negative exponent: random sweep over six decades, both cut-off conventions, with
    and without the floor, plus quotients placed on and next to whole numbers."""
    g = torch.Generator().manual_seed(5)
    N, H = 4000, 8
    a = -torch.exp(torch.empty(N, H).uniform_(math.log(1e-4), math.log(1e2), generator=g))
    rvlen = torch.exp(torch.empty(7, 3).uniform_(math.log(0.05), math.log(3.0), generator=g))
    batch = torch.randint(0, 7, (N,), generator=g)
    for cutoff, lr, mr in ((-3.5, 2, 2), (-3.5, 2, 0), (6.0, 1, 0), (-1.0, 3, 3), (0.0, 2, 0)):
        got = host_ranges(host, a, rvlen, batch, cutoff, lr, mr)
        ref = ks.translation_ranges(a, rvlen, batch, cutoff, lr, mr)
        ok = ref <= host.host_max_range()                         # (the oracle has no upper clamp)
        assert torch.equal(got[ok], ref[ok]) and int(ok.sum()) > 0.9 * ok.numel()
        assert int(got.max()) <= host.host_max_range() and int(got.min()) >= 0
    # whole-number quotients: (cutoff + 0.01) rvl / (2 pi_f) = m exactly or one ulp to either side
    two_pi = 2.0 * float(torch.tensor(3.141592654, dtype=torch.float32))
    cut = 4.0
    cases = []
    for m in range(1, 40):
        rv = torch.tensor(m * two_pi / (cut + 0.01), dtype=torch.float32)
        for step in (-2, -1, 0, 1, 2):
            r = rv.clone()
            for _ in range(abs(step)):
                r = torch.nextafter(r, torch.tensor(float("inf") if step > 0 else 0.0))
            cases.append(r)
    rv3 = torch.stack(cases)[:, None].expand(-1, 3).contiguous()
    aa = torch.full((rv3.shape[0], 1), -0.3)
    bb = torch.arange(rv3.shape[0])
    assert torch.equal(host_ranges(host, aa, rv3, bb, cut, 2, 0), ks.translation_ranges(aa, rv3, bb, cut, 2, 0))


def test_range_rule_is_bounded_on_inputs_no_model_produces(host):
    """a >= 0 (the square root of a negative number), a -> 0- (a huge cut-off), NaN, +-inf, and
    reciprocal lengths of 0, inf or NaN: every half-width stays in [max(0, floor), 64], so a kernel's
    loops over a box always end (cf_max_translation_range)."""
    inf, nan = float("inf"), float("nan")
    odd_a = torch.tensor([0.0, -0.0, 1.0, 3e38, -1e-38, -1e-45, -3e38, inf, -inf, nan, -0.3])
    odd_rv = torch.tensor([0.0, 1e-30, 0.9, 1e30, inf, nan, -1.0])
    top = host.host_max_range()
    assert top == 64
    for rv in odd_rv.tolist():
        rvlen = torch.tensor([[rv, 0.9, rv]])
        a = odd_a[:, None].contiguous()
        batch = torch.zeros(a.shape[0], dtype=torch.long)
        for cutoff, mr in ((-3.5, 0), (-3.5, 2), (4.0, 0), (inf, 0), (nan, 1)):
            R = host_ranges(host, a, rvlen, batch, cutoff, 2, mr)
            assert int(R.min()) >= mr and int(R.max()) <= top, (rv, cutoff, mr, R.flatten().tolist())
    # the sigma rule with a >= 0 or NaN: sqrt(-0.5 / a) is NaN or inf, the box is the largest one
    R = host_ranges(host, torch.tensor([[1.0], [nan], [0.0]]), torch.tensor([[0.9, 0.9, 0.9]]),
                    torch.zeros(3, dtype=torch.long), -3.5, 2, 0)
    assert R.tolist() == [[[top] * 3]] * 3
    # a -> 0-: the cut-off grows without bound and is clamped, never wrapped
    R = host_ranges(host, torch.tensor([[-1e-30], [-1e-45]]), torch.tensor([[0.9, 0.9, 0.9]]),
                    torch.zeros(2, dtype=torch.long), -3.5, 2, 0)
    assert R.tolist() == [[[top] * 3]] * 2
    # a reciprocal length of 0 gives the floor (or 0), cutoff 0 the fixed cube whatever a is
    assert host_ranges(host, torch.tensor([[-0.3]]), torch.zeros(1, 3), torch.zeros(1, dtype=torch.long),
                       -3.5, 2, 1).tolist() == [[[1, 1, 1]]]
    assert host_ranges(host, torch.tensor([[nan]]), torch.ones(1, 3), torch.zeros(1, dtype=torch.long),
                       0.0, 3, 0).tolist() == [[[3, 3, 3]]]


@pytest.mark.parametrize("sizes", [[1], [3, 1, 5, 2], [2, 0, 4, 0, 1], [64, 1, 17], [0, 0, 3]])
def test_layout_index_math_is_bit_exact(host, sizes):
    """Edge list, row offsets, crystal index per atom and pair list from the kernels' own index
    functions, against the torch-path oracle (get_edge_index) and brute force; crystals without
    atoms in any position."""
    sz = torch.tensor(sizes, dtype=torch.long)
    B, N, E = len(sizes), int(sz.sum()), int((sz * sz).sum())
    U = (E + N) // 2
    starts = torch.zeros((3, B + 1), dtype=torch.long)
    e_start = torch.zeros(N + 1, dtype=torch.long)
    edges = torch.full((2, E), -1, dtype=torch.long)
    pairs = torch.full((U, 5), -1, dtype=torch.long)
    batch = torch.full((N,), -1, dtype=torch.long)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = host.host_batch_layout(p(sz), ctypes.c_int64(B), ctypes.c_int64(N), ctypes.c_int64(E), p(starts[0]),
                                p(starts[1]), p(starts[2]), p(e_start), p(edges), p(pairs), p(batch))
    assert rc == 0
    ref_edges = tp.get_edge_index(sz)
    assert torch.equal(edges, ref_edges)
    assert torch.equal(batch, torch.repeat_interleave(torch.arange(B), sz))
    assert torch.equal(e_start, tp.edge_row_offsets(ref_edges, N))
    assert torch.equal(starts[0], torch.cat([torch.zeros(1, dtype=torch.long), sz.cumsum(0)]))
    # every edge in exactly one unit with its reverse, units in row-major order of the upper triangles
    seen = torch.zeros(E, dtype=torch.long)
    expect = []
    a0 = e0 = 0
    for b, n in enumerate(sizes):
        for i in range(n):
            for j in range(i, n):
                expect.append([e0 + i * n + j, e0 + j * n + i, a0 + i, a0 + j, b])
        a0 += n
        e0 += n * n
    assert pairs.tolist() == expect
    seen.index_add_(0, pairs[:, 0], torch.ones(U, dtype=torch.long))
    off = pairs[:, 0] != pairs[:, 1]
    seen.index_add_(0, pairs[off, 1], torch.ones(int(off.sum()), dtype=torch.long))
    assert bool((seen == 1).all())


def test_oracle_and_host_rules_run_clean_under_sanitizers():
    """AddressSanitizer + UBSan build of the C oracle and of the host rules, run on small problems
    (single atoms, empty crystals, bias only, adaptive boxes, odd exponents): no report, status 0."""
    subprocess.check_call(["make", "-C", HOST, "-B", "san_driver"], stdout=subprocess.DEVNULL,
                          stderr=subprocess.DEVNULL)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    res = subprocess.run([os.path.join(HOST, "san_driver")], capture_output=True, text=True, env=env, timeout=300)
    assert res.returncode == 0, res.stdout + res.stderr
    assert res.stdout.startswith("OK ") and "runtime error" not in res.stderr and "Sanitizer" not in res.stderr
