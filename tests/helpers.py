"""Shared test helpers: problem builders and the tolerance used for fp32 parity."""
import math

import torch

from crystalformer_amd.synthetic import make_batch
from oracle import torch_path as tp

# fp32 parity bar of this project: 1e-5 relative.  For a tensor it is applied
# against the tensor's own scale: max|x - ref| <= RTOL * max|ref|.
RTOL = 1e-5


def rel_err(x, ref):
    x = x.detach().cpu().double()
    ref = ref.detach().cpu().double()
    scale = ref.abs().max().item()
    if scale == 0.0:
        return (x - ref).abs().max().item()
    return ((x - ref).abs().max() / scale).item()


def assert_close(x, ref, what="", rtol=RTOL):
    assert x.shape == ref.shape, f"{what}: shape {tuple(x.shape)} vs {tuple(ref.shape)}"
    err = rel_err(x, ref)
    assert err <= rtol, f"{what}: relative error {err:.3e} > {rtol:.1e}"
    assert torch.isfinite(x.detach().cpu()).all(), f"{what}: non-finite values"


class Problem:
    """One encoding/attention problem on CPU tensors."""

    def __init__(self, sizes_or_batch, H=8, K=64, D=16, seed=0, W_mode="shared"):
        if isinstance(sizes_or_batch, (list, tuple)):
            b = make_sized_batch(list(sizes_or_batch), seed)
        else:
            b = sizes_or_batch
        self.b = b
        self.H, self.K, self.D = H, K, D
        self.edges = tp.get_edge_index(b.sizes)
        self.N = b.pos.shape[0]
        self.E = self.edges.shape[1]
        g = torch.Generator().manual_seed(seed + 1000)
        self.a = -(torch.rand(self.N, H, generator=g) * 0.5 + 0.05)
        self.rpos = tp.relative_positions(b.pos, self.edges)
        rec, _ = tp.reciprocal_vectors(b.trans_vec)
        self.rvlen = torch.norm(rec, 2, dim=-1)
        self.e_start = tp.edge_row_offsets(self.edges, self.N)
        self.dist_max, self.wscale = 14.0, 1.0
        self.W = None
        if K > 0:
            lead = {"shared": 1, "edge": self.E, "atom": self.N}[W_mode]
            self.W = torch.randn(lead, H, D, K, generator=g) * (K ** -0.5)
        self.g = g

    def randn(self, *shape):
        return torch.randn(*shape, generator=self.g)


def make_sized_batch(sizes, seed=0):
    """Batch with prescribed atoms per crystal."""
    b = make_batch(len(sizes), (1, 1), False, (3.0, 8.0), (70.0, 110.0), seed=seed)
    g = torch.Generator().manual_seed(seed + 7)
    sizes_t = torch.tensor(sizes, dtype=torch.long)
    N = int(sizes_t.sum())
    batch = torch.repeat_interleave(torch.arange(len(sizes)), sizes_t)
    frac = torch.rand(N, 3, generator=g)
    pos = (frac[:, None, :] @ b.trans_vec[batch]).squeeze(1).contiguous()
    Z = torch.randint(1, 95, (N,), generator=g)
    x = torch.eye(98)[Z - 1]
    from crystalformer_amd.synthetic import CrystalBatch
    return CrystalBatch(x, pos, batch, b.trans_vec, sizes_t, torch.randn(len(sizes), generator=g))


def to_dev(dev, *tensors):
    return [None if t is None else t.to(dev) for t in tensors]
