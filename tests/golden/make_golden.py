"""Writes the golden fixtures of tests/golden/ by running the REFERENCE's own
PyTorch path (CPU) on tiny seeded inputs.

Run in the build container only (the reference checkout never travels):

    python tests/golden/make_golden.py [/root/reference]

It pins what no closed form can: the RNG-ordered parameter initialisation, the
end-to-end forward of the stacked blocks with the batch-statistics
normalisation of the Gaussian exponents, the one-time write of ``gauss_scale``
in training mode, and parameter gradients of one L1 step.  Outputs are small
``.pt`` files holding tensors only (loadable with ``weights_only=True``) plus a
JSON of per-tensor SHA-256 digests for the full-size default model.
"""
from __future__ import annotations

import contextlib
import hashlib
import io
import json
import os
import sys
from types import SimpleNamespace

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, REPO)

from crystalformer_amd.latticeformer import DEFAULT_MODEL_PARAMS  # noqa: E402  (plain dict of JSON defaults)
from crystalformer_amd.synthetic import make_batch  # noqa: E402


def reference_model(ref_root: str, cfg: SimpleNamespace, seed: int):
    if ref_root not in sys.path:
        sys.path.insert(0, ref_root)
    cwd = os.getcwd()
    os.chdir(ref_root)
    try:
        from models.latticeformer import Latticeformer
        torch.manual_seed(seed)
        with contextlib.redirect_stdout(io.StringIO()):
            model = Latticeformer(cfg)
    finally:
        os.chdir(cwd)
    return model


def digest(t: torch.Tensor) -> str:
    return hashlib.sha256(t.detach().contiguous().cpu().numpy().tobytes()).hexdigest()


SMALL = dict(num_layers=2, model_dim=32, head_num=4, ff_dim=64, embedding_dim=[16], value_pe_dist_real=16,
             lattice_range=1, scale_real=[1.4, 2.0], use_cuda_code=False)


def small_cfg(**kw):
    cfg = dict(DEFAULT_MODEL_PARAMS)
    cfg.update(SMALL)
    cfg.update(kw)
    return SimpleNamespace(**cfg)


def tiny_batch(seed=3):
    b = make_batch(3, (1, 5), False, (3.0, 6.0), (75.0, 105.0), seed=seed, with_targets=True)
    return b


def run_case(ref_root: str, name: str, cfg, batch, seed: int, out: dict):
    model = reference_model(ref_root, cfg, seed)
    out[f"{name}.state"] = {k: v.detach().clone() for k, v in model.state_dict().items()}
    model.eval()
    captured = {}
    hooks = []
    for li, layer in enumerate(model.encoder.layers):
        hooks.append(layer.self_attn.register_forward_hook(
            lambda m, i, o, li=li: captured.__setitem__(f"layer{li}.values", None if o[1] is None else o[1].detach().clone())))
        hooks.append(layer.register_forward_hook(
            lambda m, i, o, li=li: captured.__setitem__(f"layer{li}.out", o.detach().clone())))
    with torch.no_grad(), contextlib.redirect_stdout(io.StringIO()):
        y = model(batch)
    for h in hooks:
        h.remove()
    out[f"{name}.eval.y"] = y.detach().clone()
    out[f"{name}.eval.gauss_scale_after"] = model.encoder.layers[0].self_attn.gauss_scale.detach().clone()
    for k, v in captured.items():
        if v is not None:
            out[f"{name}.eval.{k}"] = v
    # one training-mode forward/backward: L1 loss against the synthetic targets
    model.train()
    model.zero_grad()
    with contextlib.redirect_stdout(io.StringIO()):
        y = model(batch)
    loss = torch.nn.functional.l1_loss(y.squeeze(-1), batch.y)
    loss.backward()
    out[f"{name}.train.y"] = y.detach().clone()
    out[f"{name}.train.loss"] = loss.detach().clone()
    out[f"{name}.train.grads"] = {k: p.grad.detach().clone() for k, p in model.named_parameters()
                                  if p.grad is not None}
    out[f"{name}.train.gauss_scale_after"] = torch.stack(
        [l.self_attn.gauss_scale.detach().clone() for l in model.encoder.layers])
    # a second eval forward now uses the stored scales
    model.eval()
    with torch.no_grad(), contextlib.redirect_stdout(io.StringIO()):
        out[f"{name}.eval2.y"] = model(batch).detach().clone()


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    torch.set_num_threads(1)
    out = {}
    batch = tiny_batch()
    out["batch"] = {"x": batch.x, "pos": batch.pos, "batch": batch.batch, "trans_vec": batch.trans_vec,
                    "sizes": batch.sizes, "y": batch.y}
    run_case(ref_root, "k16_r1", small_cfg(), batch, 11, out)
    run_case(ref_root, "k0_r2", small_cfg(value_pe_dist_real=0, lattice_range=2), batch, 12, out)
    torch.save(out, os.path.join(HERE, "reference_small_model.pt"))

    # reciprocal-space blocks: alternating real / reciprocal layers, and half-and-half heads
    out = {"batch": out["batch"]}
    run_case(ref_root, "real_reci_k16_r1", small_cfg(domain="real-reci"), batch, 13, out)
    run_case(ref_root, "multihead_k0_r2", small_cfg(domain="multihead", value_pe_dist_real=0, lattice_range=2),
             batch, 14, out)
    run_case(ref_root, "reci_r2", small_cfg(domain="reci", value_pe_dist_real=0, lattice_range=2), batch, 15, out)
    torch.save(out, os.path.join(HERE, "reference_small_model_reciprocal.pt"))

    # full-size default model: digests of the seeded initial parameters only
    cfg = SimpleNamespace(**dict(DEFAULT_MODEL_PARAMS, use_cuda_code=False))
    model = reference_model(ref_root, cfg, 123)
    digests = {k: {"sha256": digest(v), "shape": list(v.shape)} for k, v in model.state_dict().items()}
    digests["__num_parameters__"] = sum(p.numel() for p in model.parameters())
    with open(os.path.join(HERE, "reference_default_init_sha256.json"), "w") as f:
        json.dump(digests, f, indent=1, sort_keys=True)
    print("wrote", os.listdir(HERE))


if __name__ == "__main__":
    main()
