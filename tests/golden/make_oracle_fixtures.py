"""Writes the CPU oracle's results for the benchmark configurations whose dense CPU
evaluation takes minutes (7-block forward at 256 crystals, training step at 128 crystals,
4-block forward on 200+-atom cells), so that the GPU parity tests compare against them
without re-running the oracle every time:

    python tests/golden/make_oracle_fixtures.py            # all four, about fifteen minutes on 8 cores

Nothing of the reference is imported or read: inputs come from the package's own seeded
generator (crystalformer_amd/synthetic.py) and seeded parameter initialisation, results
from oracle/torch_model.py (float32, the fixed translation cube).  Each file stores a
SHA-256 digest of its inputs and parameters; the tests rebuild both and refuse a fixture
whose digest does not match (a changed generator or initialisation needs a re-run).
"""
import hashlib
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from crystalformer_amd.latticeformer import Latticeformer, default_params          # noqa: E402
from crystalformer_amd.synthetic import CONFIGS, make_config_batch, select_crystals  # noqa: E402
from oracle import torch_model as om                                               # noqa: E402
from oracle import torch_path as tp                                                # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
SAMPLE_STRIDE = 37          # per-layer outputs are kept for every 37th atom


def digest(batch, state) -> str:
    h = hashlib.sha256()
    for t in (batch.x, batch.pos, batch.batch, batch.trans_vec, batch.sizes, batch.y):
        if t is not None:
            h.update(t.contiguous().numpy().tobytes())
    for k in sorted(state):
        h.update(k.encode())
        h.update(state[k].detach().contiguous().numpy().tobytes())
    return h.hexdigest()


def build(name, seed=1, **over):
    cfg = default_params(**{**CONFIGS[name]["model"], "adaptive_cutoff_sigma": 0.0, **over})
    torch.manual_seed(seed)
    return cfg, Latticeformer(cfg)


def cfg5_subset(batch):
    """The two smallest of the 200..444-atom cells (keeps the dense CPU evaluation to a minute)."""
    order = torch.argsort(batch.sizes, stable=True)[:2].sort().values
    return select_crystals(batch, order.tolist())


def forward_fixture(name, batch, tag):
    cfg, model = build(name)
    state = {k: v.detach().clone() for k, v in model.state_dict().items()}
    cap = {}
    t = time.time()
    with torch.no_grad():
        y = om.latticeformer_forward(state, cfg, batch, capture=cap)
    sel = torch.arange(0, batch.pos.shape[0], SAMPLE_STRIDE)
    out = {"digest": digest(batch, {k: v for k, v in model.state_dict().items()}), "y": y, "atoms": sel,
           "pooled": cap["pooled"]}
    for li in range(cfg.num_layers):
        out[f"layer{li}.out"] = cap[f"layer{li}.out"][sel].clone()
        out[f"layer{li}.alpha"] = cap[f"layer{li}.alpha"][sel].clone()
    torch.save(out, os.path.join(HERE, f"oracle_{tag}.pt"))
    print(f"{tag}: {time.time() - t:.0f} s, N={batch.pos.shape[0]}, E={batch.num_edges}")


RELU_MARGIN = 2e-6


def kink_free_shift(h, margin):
    """Per hidden unit (column of ``h``) the smallest shift s with |h + s| >= margin for every row."""
    import numpy as np
    hv = h.detach().double().numpy()
    out = np.zeros(hv.shape[1])
    for u in range(hv.shape[1]):
        v = np.sort(hv[:, u])
        # t = -s must keep clear of every value: outside all intervals [v - margin, v + margin]
        cands = np.concatenate([[0.0], v - margin * 1.0001, v + margin * 1.0001])
        cands = cands[np.argsort(np.abs(cands))]
        for t in cands[:64]:
            k = np.searchsorted(v, t)
            lo = v[k - 1] if k > 0 else -np.inf
            hi = v[k] if k < v.size else np.inf
            if t - lo >= margin and hi - t >= margin:
                out[u] = -t
                break
        else:
            raise RuntimeError(f"no kink-free shift for unit {u}")
    return torch.from_numpy(out)


def settle_relu_kinks(state, cfg, b64, margin=RELU_MARGIN):
    """A ReLU whose argument is zero to eight digits makes the gradient a matter of rounding: a
    float32 evaluation and this float64 one then legitimately disagree on one hidden unit's mask,
    and through it on a whole row of a weight gradient (about one atom in 1774, i.e. 1e-2 of the
    row).  With about 60 of the 908,288 pre-activations of a block within 1e-6 of zero at random
    initialisation, that happens in every other run.  The comparison is only defined away from
    the kinks, so the first feed-forward bias of every block (zero at initialisation) is moved by
    the smallest amount (a few 1e-5, against pre-activations of order 1e-2) that leaves no
    pre-activation of the batch within ``margin`` of zero.  Returns the adjusted biases (float32);
    ``state`` is updated in place."""
    import torch.nn.functional as F
    P = {k: v.double() for k, v in state.items()}
    adjusted = {}
    with torch.no_grad():
        x = F.linear(b64.x, P["input_embeddings.weight"])
        batch = b64.batch - b64.batch[0]
        sizes_l = b64.sizes.tolist()
        edges = tp.get_edge_index(sizes_l)
        for layer in range(cfg.num_layers):
            lp = f"encoder.layers.{layer}."
            x = x + om.attention_block(P, lp + "self_attn.", cfg, layer, x, b64.pos, batch, b64.trans_vec, sizes_l,
                                       edges, True)
            name = lp + "linear1.bias"
            for _ in range(3):          # the shift is rounded to float32 with the bias: check, and repeat if needed
                h = F.linear(x, P[lp + "linear1.weight"], P[name])
                if float(h.abs().min()) >= margin:
                    break
                P[name] = (P[name] + kink_free_shift(h, margin * 1.5)).float().double()
            assert float(h.abs().min()) >= margin, (layer, float(h.abs().min()))
            adjusted[name] = P[name].float()
            x = x + F.linear(F.relu(h), P[lp + "linear2.weight"], P[lp + "linear2.bias"])
    for name, v in adjusted.items():
        state[name] = v.clone()
    return adjusted


def train_fixture(name, tag):
    """One training-mode forward, the reference's step loss (models/regression.py:117-118 with
    losses/regression_loss.py:17-20) and its backward: every parameter gradient, and the
    batch statistics the training-mode forward stores in ``gauss_scale``.  Evaluated in float64
    on the float32 inputs and parameters (about 40 GB of autograd state): gradients are long sums
    with cancellation, and a float32 CPU evaluation would carry as much rounding as the kernels
    it is there to check.  Parameters are the seeded initialisation except for the first
    feed-forward biases, see :func:`settle_relu_kinks`; the test loads ``adjusted`` on top of its
    own seeded model."""
    cfg, model = build(name)
    batch = make_config_batch(name)
    state0 = {k: v.detach().clone() for k, v in model.state_dict().items()}
    dig = digest(batch, state0)
    b64 = type(batch)(batch.x.double(), batch.pos.double(), batch.batch, batch.trans_vec.double(), batch.sizes,
                      batch.y.double())
    t = time.time()
    adjusted = settle_relu_kinks(state0, cfg, b64)
    print(f"{tag}: biases settled after {time.time() - t:.0f} s, largest shift "
          f"{max(float(v.abs().max()) for v in adjusted.values()):.2e}", flush=True)
    P = {k: v.detach().double().requires_grad_("scale" not in k) for k, v in state0.items()}
    y = om.latticeformer_forward(P, cfg, b64, training=True)
    loss = tp.l1_training_loss(y, b64.y.reshape(-1, 1))
    loss.backward()
    out = {"digest": dig, "adjusted": adjusted, "relu_margin": torch.tensor(RELU_MARGIN),
           "y": y.detach().float(), "loss": loss.detach().float(),
           "grads": {k: v.grad.float() for k, v in P.items() if v.grad is not None},
           "gauss_scale_after": torch.stack([P[f"encoder.layers.{li}.self_attn.gauss_scale"].detach()
                                             for li in range(cfg.num_layers)]).float()}
    torch.save(out, os.path.join(HERE, f"oracle_{tag}.pt"))
    print(f"{tag}: {time.time() - t:.0f} s")


if __name__ == "__main__":
    which = sys.argv[1:] or ["cfg3", "cfg4", "cfg5", "cfg5full"]
    if "cfg5full" in which:         # all 16 cells of 200..444 atoms, 1.77 M edges: about five minutes on 8 cores
        forward_fixture("cfg5_stress_b16", make_config_batch("cfg5_stress_b16"), "cfg5_forward")
    if "cfg5" in which:
        forward_fixture("cfg5_stress_b16", cfg5_subset(make_config_batch("cfg5_stress_b16")), "cfg5_subset_forward")
    if "cfg4" in which:
        train_fixture("cfg4_train_b128", "cfg4_train_step")
    if "cfg3" in which:
        forward_fixture("cfg3_7block_b256", make_config_batch("cfg3_7block_b256"), "cfg3_forward")
