"""CPU-side checks of the boundary: the shared object loads, exports every
symbol the public header declares, rejects bad arguments before touching a
device, and the host-side helpers (parameter bag, synthetic crystals, operator
front-ends) behave as the reference's do.  No compute call is made here."""
import ctypes
import os
import re
from types import SimpleNamespace

import pytest
import torch

from crystalformer_amd import hip_funcs, lib, ops
from crystalformer_amd.params import LatticeformerParams
from crystalformer_amd.synthetic import CONFIGS, make_batch, make_config_batch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "crystalformer_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cf_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 14 and "cf_edge_pairs" in names and "cf_real_enc_fwd" in names and "cf_fused_dpa_bwd" in names
    L = lib.load()
    for n in names:
        assert hasattr(L, n), f"{n} declared in the header but not exported"
    assert set(names) == set(lib.SIGNATURES), "python signatures out of sync with the header"
    assert L.cf_version() >= 100
    assert L.cf_max_translation_range() == 64


def test_argument_validation_needs_no_device():
    L = lib.load()
    null = ctypes.c_void_p(0)
    # unsupported head count
    rc = L.cf_real_enc_fwd(null, null, null, null, null, 0, 3, 0, 0, 0, 0, 1.0, 1.0, null, 0, null, 0.0, 2, 0,
                           null, 0, null, null, null, null)
    assert rc == -2 and b"head count" in L.cf_last_error()
    # K outside range
    rc = L.cf_real_enc_fwd(null, null, null, null, null, 0, 8, 0, 0, 500, 16, 1.0, 1.0, null, 0, null, 0.0, 2, 0,
                           null, 0, null, null, null, null)
    assert rc == -2 and b"K=" in L.cf_last_error()
    # adaptive cut-off without reciprocal lengths
    rc = L.cf_real_enc_fwd(null, null, null, null, null, 0, 8, 0, 0, 0, 0, 1.0, 1.0, null, 0, null, -3.5, 2, 0,
                           null, 0, null, null, null, null)
    assert rc == -1 and b"rvlen" in L.cf_last_error()
    # null pointers with work to do
    rc = L.cf_real_enc_fwd(null, null, null, null, null, 4, 8, 16, 1, 0, 0, 1.0, 1.0, null, 0, null, 0.0, 2, 0,
                           null, 0, null, null, null, null)
    assert rc == -1
    rc = L.cf_fused_dpa_fwd(null, null, null, null, null, null, null, 4, 8, 16, 16, 16, null, null, null)
    assert rc == -1
    rc = L.cf_fused_dpa_bwd(*([null] * 9), 4, 8, 16, 1, 16, 12, *([null] * 9))
    assert rc == -2 and b"power of two" in L.cf_last_error()
    rc = L.cf_minimum_distance(null, null, null, null, 4, null, -1.0, 2, 0, null, null)
    assert rc == -1
    # empty problems are fine and launch nothing
    assert L.cf_real_enc_fwd(null, null, null, null, null, 0, 8, 0, 0, 64, 16, 14.0, 1.0, null, 1, null, 0.0, 2,
                             0, null, 0, null, null, null, null) == 0
    # a pair list must have (E + N) / 2 entries
    one = ctypes.c_void_p(8)
    rc = L.cf_real_enc_fwd(one, one, one, one, one, 4, 8, 16, 1, 64, 16, 14.0, 1.0, one, 1, null, 0.0, 2, 0,
                           one, 7, null, one, one, null)
    assert rc == -1 and b"pair list" in L.cf_last_error()
    assert L.cf_irregular_mean_fwd(null, null, 0, 128, null, null) == 0
    assert L.cf_edge_index(null, null, 0, 0, null, null, null, null) == 0
    assert L.cf_real_enc_bwd_workspace(10, 8, 100, 64, 16, 1, 1) >= 100 * 8 * 4 + 100 * 8 * 64 * 4


def test_operators_refuse_cpu_tensors():
    a = torch.zeros(2, 8)
    with pytest.raises(lib.CrystalformerHipError, match="no CPU fallback"):
        ops.real_enc_fwd(a, torch.zeros(4, 3), torch.zeros(1, 3, 3), torch.zeros(2, dtype=torch.long),
                         torch.zeros(2, 4, dtype=torch.long), 0, 1.0, 1.0)
    with pytest.raises(lib.CrystalformerHipError):
        hip_funcs.IrregularMeanCUDA.apply(torch.zeros(3, 4), torch.zeros(3, dtype=torch.long),
                                          torch.tensor([3]))


def test_compile_kernels_records_constants_and_checks_shapes():
    hip_funcs.compile_kernels(2, 8, 16, 64, 16, True)
    KM = hip_funcs.KernelManager
    assert (KM.LATTICE_RANGE, KM.MINIMUM_RANGE, KM.HEAD_NUM, KM.VPE_DIM) == (2, 2, 8, 64)
    hip_funcs.compile_kernels(3, 4, 8, 0, 8, False)
    assert (KM.LATTICE_RANGE, KM.MINIMUM_RANGE) == (3, 0)
    with pytest.raises(lib.CrystalformerHipError):
        hip_funcs.compile_kernels(2, 5, 16, 64, 16, True)
    with pytest.raises(lib.CrystalformerHipError):
        hip_funcs.compile_kernels(2, 8, 16, 512, 16, True)
    hip_funcs.compile_kernels(2, 8, 16, 64, 16, True)


def test_params_layer_resolution():
    P = LatticeformerParams(scale_real=[1.4, 2.0, 3.0], domain="real")
    assert [P.getLayerParameters(i).scale_real for i in range(5)] == [1.4, 2.0, 3.0, 1.4, 2.0]
    assert P.getLayerParameters(1).layer_index == 1 and P.scale_real == [1.4, 2.0, 3.0]
    assert LatticeformerParams().lattice_range == 4          # class default differs from the JSON's 2
    Q = LatticeformerParams()
    Q.parseFromArgs(SimpleNamespace(lattice_range=2, value_pe_dist_real=0, unrelated=1))
    assert Q.lattice_range == 2 and Q.value_pe_dist_real == 0 and not hasattr(Q, "unrelated")
    R = LatticeformerParams(domain="real-reci")
    assert [R.getLayerParameters(i).domain for i in range(3)] == ["real", "reci", "real"]


def test_synthetic_batches_follow_the_field_contract():
    b = make_batch(16, (1, 16), False, (3, 12), (70, 110), seed=0, with_targets=True)
    N = int(b.sizes.sum())
    assert b.x.shape == (N, 98) and bool((b.x.sum(1) == 1).all())
    assert b.pos.shape == (N, 3) and b.batch.shape == (N,) and b.trans_vec.shape == (16, 3, 3)
    assert b.batch.dtype == torch.long and b.sizes.dtype == torch.long
    assert torch.equal(torch.bincount(b.batch, minlength=16), b.sizes)
    assert int(b.sizes.min()) >= 1 and int(b.sizes.max()) <= 16
    lens = b.trans_vec.norm(dim=-1)
    assert float(lens.min()) >= 3 - 1e-4 and float(lens.max()) <= 12 + 1e-4
    assert bool((torch.linalg.det(b.trans_vec.double()) > 0).all())
    # fractional coordinates recovered from pos lie in [0,1)
    frac = torch.linalg.solve(b.trans_vec.double()[b.batch].transpose(1, 2), b.pos.double()[..., None]).squeeze(-1)
    assert float(frac.min()) > -1e-5 and float(frac.max()) < 1 + 1e-5
    b2 = make_batch(16, (1, 16), False, (3, 12), (70, 110), seed=0, with_targets=True)
    assert torch.equal(b.pos, b2.pos) and torch.equal(b.sizes, b2.sizes)
    assert b.num_edges == int((b.sizes ** 2).sum())


def test_benchmark_configs_have_the_stated_sizes():
    c2 = make_config_batch("cfg2_default_b128")
    assert c2.sizes.numel() == 128 and 1 <= int(c2.sizes.min()) and int(c2.sizes.max()) <= 64
    assert 4 <= float(c2.sizes.double().median()) <= 16          # log-uniform: median near 8
    c5 = make_config_batch("cfg5_stress_b16")
    assert c5.sizes.numel() == 16 and int(c5.sizes.min()) >= 200 and int(c5.sizes.max()) <= 444
    lens = c5.trans_vec.norm(dim=-1)
    assert float(lens[:, 0].min()) >= 20 and float(lens[:, 1:].max()) <= 8 + 1e-4
    assert set(CONFIGS) == {"cfg1_simplified_b32", "cfg2_default_b128", "cfg3_7block_b256", "cfg4_train_b128",
                            "cfg5_stress_b16"}
