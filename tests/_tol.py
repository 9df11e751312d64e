"""Per-element error bounds shared by the GPU parity tests.

16-bit tensors (bf16 / fp16 results against the fp32 oracle on the same rounded inputs):
an element whose reference value is at most 4 in magnitude may be off by 2e-2; above
that the bound is one bf16 ulp of the reference value, 2^-7 * |ref| (the result itself is
rounded to the element type on output, so an absolute bound cannot hold for large values).
The bound of every element depends on that element's reference value only: a large value
somewhere in the tensor does not loosen the bound of a small one.
"""
import torch

TOL_ABS = 2e-2
BIG = 4.0
REL_BIG = 2.0 ** -7


def worst_ratio(got, ref, tol_abs=TOL_ABS):
    """max over elements of |got - ref| / bound(ref); <= 1 passes.  Also returns where it sits."""
    got = torch.as_tensor(got).detach().float().cpu()
    ref = torch.as_tensor(ref).detach().float().cpu()
    assert got.shape == ref.shape, (tuple(got.shape), tuple(ref.shape))
    if ref.numel() == 0:
        return 0.0, 0.0, 0.0
    mag = ref.abs()
    bound = torch.where(mag <= BIG, torch.full_like(mag, tol_abs), mag * (REL_BIG * tol_abs / TOL_ABS))
    ratio = (got - ref).abs() / bound
    ratio = torch.where(torch.isnan(ratio), torch.full_like(ratio, float("inf")), ratio)
    idx = int(ratio.argmax())
    return float(ratio.flatten()[idx]), float((got - ref).abs().flatten()[idx]), float(ref.flatten()[idx])


def check_close(name, got, ref, tol_abs=TOL_ABS, quiet=False):
    """Assert the per-element bound and print the margin (worst |err| / bound)."""
    r, err, at = worst_ratio(got, ref, tol_abs)
    if not quiet:
        print(f"  {name}: worst err/bound {r:.3f} (err {err:.4g} at ref {at:.4g})", flush=True)
    assert r <= 1.0, f"{name}: error {err:.5g} at reference value {at:.5g} is {r:.3f} x the bound"
    return r
