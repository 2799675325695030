"""Golden vectors written by importing the reference's own PyTorch path
(tests/golden/make_golden.py): they pin what no closed form can — RNG-ordered
initialisation, the stacked-block forward with batch-statistics normalisation
of the Gaussian exponents, the one-time gauss_scale write and one L1 step's
gradients."""
import hashlib
import json
import os
import sys
from types import SimpleNamespace

import pytest
import torch

from oracle import torch_model as om
from tests.helpers import rel_err

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
sys.path.insert(0, GOLD)
from make_golden import small_cfg  # noqa: E402

CASES = [("k16_r1", dict(), 11), ("k0_r2", dict(value_pe_dist_real=0, lattice_range=2), 12)]


@pytest.fixture(scope="module")
def gold():
    return torch.load(os.path.join(GOLD, "reference_small_model.pt"), weights_only=True)


@pytest.mark.parametrize("name,over,seed", CASES)
def test_oracle_forward_matches_reference(gold, name, over, seed):
    cfg = small_cfg(**over)
    data = SimpleNamespace(**gold["batch"])
    P = {k: v.clone() for k, v in gold[f"{name}.state"].items()}
    cap = {}
    y = om.latticeformer_forward(P, cfg, data, training=False, capture=cap)
    assert rel_err(y, gold[f"{name}.eval.y"]) < 1e-6
    for li in range(cfg.num_layers):
        assert rel_err(cap[f"layer{li}.out"], gold[f"{name}.eval.layer{li}.out"]) < 1e-6
        key = f"{name}.eval.layer{li}.values"
        if key in gold:
            assert rel_err(cap[f"layer{li}.values"], gold[key]) < 1e-6
    # eval mode leaves gauss_scale untouched (batch statistics recomputed every call)
    assert float(P["encoder.layers.0.self_attn.gauss_scale"].abs().sum()) == 0.0
    assert float(gold[f"{name}.eval.gauss_scale_after"].abs().sum()) == 0.0


@pytest.mark.parametrize("name,over,seed", CASES)
def test_oracle_training_step_matches_reference(gold, name, over, seed):
    cfg = small_cfg(**over)
    data = SimpleNamespace(**gold["batch"])
    P = {k: v.clone().requires_grad_("scale" not in k) for k, v in gold[f"{name}.state"].items()}
    y = om.latticeformer_forward(P, cfg, data, training=True)
    loss = torch.nn.functional.l1_loss(y.squeeze(-1), data.y)
    loss.backward()
    assert rel_err(y, gold[f"{name}.train.y"]) < 1e-6
    assert abs(float(loss.detach()) - float(gold[f"{name}.train.loss"])) < 1e-6
    for k, g in gold[f"{name}.train.grads"].items():
        assert rel_err(P[k].grad, g) < 1e-5, k
    scales = torch.stack([P[f"encoder.layers.{l}.self_attn.gauss_scale"].detach() for l in range(cfg.num_layers)])
    assert rel_err(scales, gold[f"{name}.train.gauss_scale_after"]) < 1e-6
    # later eval forwards use the stored scales
    Pd = {k: v.detach() for k, v in P.items()}
    y2 = om.latticeformer_forward(Pd, cfg, data, training=False)
    assert rel_err(y2, gold[f"{name}.eval2.y"]) < 1e-6


@pytest.mark.parametrize("name,over,seed", CASES)
def test_host_module_initialisation_is_bit_identical(gold, name, over, seed):
    from crystalformer_amd.latticeformer import Latticeformer
    torch.manual_seed(seed)
    model = Latticeformer(small_cfg(**over))
    state = model.state_dict()
    ref = gold[f"{name}.state"]
    assert list(state.keys()) == list(ref.keys())
    for k in ref:
        assert state[k].shape == ref[k].shape and torch.equal(state[k], ref[k]), k


def test_default_model_initialisation_digests():
    from crystalformer_amd.latticeformer import DEFAULT_MODEL_PARAMS, Latticeformer
    with open(os.path.join(GOLD, "reference_default_init_sha256.json")) as f:
        ref = json.load(f)
    torch.manual_seed(123)
    model = Latticeformer(SimpleNamespace(**DEFAULT_MODEL_PARAMS))
    assert sum(p.numel() for p in model.parameters()) == ref.pop("__num_parameters__") == 853517
    state = model.state_dict()
    assert sorted(state.keys()) == sorted(ref.keys())
    for k, v in state.items():
        assert list(v.shape) == ref[k]["shape"]
        assert hashlib.sha256(v.detach().contiguous().numpy().tobytes()).hexdigest() == ref[k]["sha256"], k


def test_optional_parameters_of_the_attention_module():
    """Options off the default path that add parameters, as the reference's kernel-path module lays them
    out (models/indexed_lattice_multi_head_attention_cuda.py:855-878, 894-947): the plane-wave projection
    is created and initialised after the distance projection (it has no effect on that module's output,
    and none here), gauss_state "x-xn" has two factors.  Parameters drawn before the new ones keep the
    values of the default model (same random stream up to there), and the golden initialisation of
    the default configuration is untouched."""
    import warnings
    from crystalformer_amd.latticeformer import Latticeformer
    torch.manual_seed(7)
    base = Latticeformer(small_cfg()).state_dict()
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        torch.manual_seed(7)
        waves = Latticeformer(small_cfg(value_pe_wave_real=2)).state_dict()
    assert any("pe_wave_proj" in str(w.message) for w in caught)
    key = "encoder.layers.0.self_attn.pe_wave_proj"
    dist = "encoder.layers.0.self_attn.pe_dist_proj"
    assert waves[key].shape == (1, base[dist].shape[1], base[dist].shape[2], 8)
    assert float(waves[key].abs().max()) > 0
    keys = list(waves.keys())
    assert keys.index(key) == keys.index(dist) + 1
    for k in ("input_embeddings.weight", "encoder.layers.0.self_attn.q_proj_weight", dist,
              "encoder.layers.0.self_attn.lattice_pos_weights"):
        assert torch.equal(waves[k], base[k]), k
    torch.manual_seed(7)
    two = Latticeformer(small_cfg(gauss_state="x-xn"))
    attn = two.encoder.layers[0].self_attn
    H, D = attn.num_heads, attn.embed_dim
    assert attn.lattice_pos_weights.shape == (attn.kdim, D) and attn.lattice_pos_weights2.shape == (attn.kdim,)
    assert attn.position_weights().shape == (H, D)
    torch.manual_seed(7)
    one = Latticeformer(small_cfg(gauss_state="x-xn2")).encoder.layers[0].self_attn
    # "x-xn2" is the product of the same two factors, drawn once at initialisation
    assert torch.equal(one.lattice_pos_weights, attn.position_weights())


# ------------------------------------------------- reciprocal-space blocks
RECI_CASES = [("real_reci_k16_r1", dict(domain="real-reci"), 13),
              ("multihead_k0_r2", dict(domain="multihead", value_pe_dist_real=0, lattice_range=2), 14),
              ("reci_r2", dict(domain="reci", value_pe_dist_real=0, lattice_range=2), 15)]


@pytest.fixture(scope="module")
def gold_reci():
    return torch.load(os.path.join(GOLD, "reference_small_model_reciprocal.pt"), weights_only=True)


@pytest.mark.parametrize("name,over,seed", RECI_CASES)
def test_oracle_reciprocal_blocks_match_reference(gold_reci, name, over, seed):
    """Alternating real / reciprocal layers, half-and-half heads and all-reciprocal blocks:
    the oracle's forward, per-layer outputs and one L1 step's gradients (autograd, i.e. with
    the normalisation term's derivative, as on the reference's PyTorch path)."""
    gold = gold_reci
    cfg = small_cfg(**over)
    data = SimpleNamespace(**gold["batch"])
    P = {k: v.clone() for k, v in gold[f"{name}.state"].items()}
    cap = {}
    y = om.latticeformer_forward(P, cfg, data, training=False, capture=cap)
    assert rel_err(y, gold[f"{name}.eval.y"]) < 2e-6
    for li in range(cfg.num_layers):
        assert rel_err(cap[f"layer{li}.out"], gold[f"{name}.eval.layer{li}.out"]) < 2e-6
        key = f"{name}.eval.layer{li}.values"
        assert (key in gold) == (f"layer{li}.values" in cap)
        if key in gold:
            assert rel_err(cap[f"layer{li}.values"], gold[key]) < 1e-6
    P = {k: v.clone().requires_grad_("scale" not in k) for k, v in gold[f"{name}.state"].items()}
    y = om.latticeformer_forward(P, cfg, data, training=True)
    loss = torch.nn.functional.l1_loss(y.squeeze(-1), data.y)
    loss.backward()
    assert abs(float(loss.detach()) - float(gold[f"{name}.train.loss"])) < 1e-6
    for k, g in gold[f"{name}.train.grads"].items():
        assert rel_err(P[k].grad, g) < 2e-5, k


@pytest.mark.parametrize("name,over,seed", RECI_CASES)
def test_host_module_initialisation_with_reciprocal_blocks(gold_reci, name, over, seed):
    from crystalformer_amd.latticeformer import Latticeformer
    torch.manual_seed(seed)
    state = Latticeformer(small_cfg(**over)).state_dict()
    ref = gold_reci[f"{name}.state"]
    assert list(state.keys()) == list(ref.keys())
    for k in ref:
        assert state[k].shape == ref[k].shape and torch.equal(state[k], ref[k]), k
