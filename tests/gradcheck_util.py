"""Gradient comparison used by the GPU parity tests.

The path's stated tolerance is a whole-tensor relative norm of 5e-2.  The kernels achieve
about 3e-3 with bf16 inputs, and a whole-tensor norm hardly moves when a single row is wrong
(one zeroed row of 400 changes it by 5 %), so the tests hold the kernels to a bound close to
what they achieve and add an elementwise check that one bad row or one boundary key fails:

  * whole tensor:  ||x - ref|| <= GRAD_TOL * ||ref||                      (GRAD_TOL = 1e-2)
  * elementwise:   |x - ref|  <= ELEM_ATOL * max|ref| + ELEM_RTOL * |ref|   (2e-2, 2e-2)

The absolute floor scales with the tensor's largest entry, which keeps rows with a single
visible key (tiny gradients, large relative rounding) from failing on noise.
"""
import torch

GRAD_TOL = 1e-2
ELEM_ATOL = 2e-2
ELEM_RTOL = 2e-2


def elementwise_close(x, ref, name="gradient"):
    x = x.detach().float().cpu()
    ref = ref.detach().float().cpu()
    if not ref.numel():
        return
    # absolute floor for tensors whose exact value is (almost) zero everywhere
    bound = ELEM_ATOL * ref.abs().max() + ELEM_RTOL * ref.abs() + 1e-4
    bad = (x - ref).abs() > bound
    if bad.any():
        idx = bad.nonzero()[0].tolist()
        raise AssertionError(
            f"{name}: {int(bad.sum())} of {bad.numel()} entries off by more than "
            f"{ELEM_ATOL} * max|ref| + {ELEM_RTOL} * |ref|; first at {idx}: "
            f"{x[tuple(idx)].item()} vs {ref[tuple(idx)].item()}")


def relnorm(x, ref, elementwise=True):
    """Relative norm of the error; asserts the elementwise bound on the way."""
    x = x.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert x.shape == ref.shape, f"{tuple(x.shape)} vs {tuple(ref.shape)}"
    assert not torch.isnan(x).any(), "NaN in a gradient"
    den = ref.norm().item()
    if elementwise:
        elementwise_close(x, ref)
    if den == 0.0:
        return x.norm().item()
    return (x - ref).norm().item() / den
