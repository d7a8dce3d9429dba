"""The product's batched Newton-Schulz (torch path) against the oracle's literal formula in fp64.

``pylo_amd.optim.ELO_CELO2_cuda.newton_schulz`` associates the quintic differently from
pylo/optim/CELO2_naive.py:59-73 -- (c2 A + c1 I) A and (B + c0 I) X, tall matrices untransposed, the
Gram product of a very tall matrix cut into row slabs -- so each of those branches is compared with the
oracle evaluated in fp64 at the rel 1e-5 / abs 1e-6 bar.  Runs on the CPU: the function is plain torch.
"""

import pytest
import torch

from golden_io import max_err
from oracle import pylo_oracle as O
from pylo_amd.optim.ELO_CELO2_cuda import _gram_split, newton_schulz

COEFFS = (3.4445, -4.7750, 2.0315)


@pytest.mark.parametrize("shape,split", [
    ((2, 16384, 64), 32),      # very tall: the slab Gram product
    ((2, 64, 16384), 1),       # its wide counterpart
    ((3, 96, 40), 1),          # tall, one slab
    ((3, 40, 96), 1),          # wide
    ((1, 48, 48), 1),          # square
    ((2, 3, 24, 56), 1),       # more leading dims: one batch of matrices
])
def test_batched_newton_schulz_matches_the_literal_formula(shape, split):
    tall = shape[-2] > shape[-1]
    long_dim, small = max(shape[-2:]), min(shape[-2:])
    batch = 1
    for s in shape[:-2]:
        batch *= s
    if tall:                      # slabs are taken for tall matrices only
        assert _gram_split(long_dim, small, batch) == split
    gen = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(shape, generator=gen) * 3e-3
    want = O.newton_schulz(x.double(), COEFFS, 5, 1e-8)
    got = newton_schulz(x, COEFFS, 5, 1e-8)
    assert got.shape == x.shape and got.dtype == torch.float32
    assert max_err(got, want, 1e-5, 1e-6) <= 1.0
    # the literal fp32 formula is no closer to fp64 than a few of its own rounding errors
    lit = O.newton_schulz(x, COEFFS, 5, 1e-8)
    assert max_err(got, lit, 1e-5, 1e-6) <= 1.0
    if tall and split > 1:
        # the slab sum is the Gram matrix: one iteration's A against the plain product
        xs = (x / (torch.linalg.norm(x, dim=(-2, -1), keepdim=True) + 1e-8)).double()
        a_plain = xs.transpose(-2, -1) @ xs
        parts = xs.reshape(shape[0] * split, shape[1] // split, shape[2])
        a_slab = torch.bmm(parts.transpose(-2, -1), parts).view(shape[0], split, shape[2], shape[2]).sum(1)
        assert torch.allclose(a_plain, a_slab, rtol=1e-12, atol=1e-15)
