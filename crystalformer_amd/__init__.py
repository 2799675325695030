"""MI355X-native implementation of Crystalformer's infinitely connected
attention: real-space periodic encoding, fused edge-indexed attention and
irregular per-crystal reductions as gfx950 HIP kernels behind the reference's
operator interface."""

__version__ = "0.1.0"
