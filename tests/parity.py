"""The parity bar of the layer-level GPU tests.

Target: rel 1e-5 / abs 1e-6 against the reference's fp32 math.  That math (sums over 30-200 edges, K = 512
reductions, group norms) evaluated in fp32 is itself some distance `e_ref` from exact arithmetic, and that distance
depends on the summation order, which the reference does not fix (atomics, shuffles, BLAS).  So every check
evaluates the oracle twice, in float32 and in float64, and accepts the HIP result iff, elementwise,

    |hip - f64| <= 1e-6 + 1e-5 |f64| + 2 e_ref,        e_ref = max |f32 oracle - f64 oracle|

i.e. the stated tolerance widened by nothing but twice the measured rounding error of the fp32 reference math on the
same inputs.  The measured e_ref and e_hip = max |hip - f64| are printed (run pytest with -s to collect them).
"""
import torch


def assert_parity(got, ref32, ref64, what="", rtol=1e-5, atol=1e-6, slack=2.0):
    got = got.detach().cpu().double()
    ref64 = ref64.detach().cpu().double()
    ref32 = ref32.detach().cpu().double()
    assert got.shape == ref64.shape == ref32.shape, (got.shape, ref32.shape, ref64.shape)
    e_ref = float((ref32 - ref64).abs().max()) if ref64.numel() else 0.0
    err = (got - ref64).abs()
    e_hip = float(err.max()) if ref64.numel() else 0.0
    scale = float(ref64.abs().max()) if ref64.numel() else 0.0
    print(f"[parity] {what}: scale {scale:.3g}  e_ref(fp32 oracle vs f64) {e_ref:.3g}  e_hip(vs f64) {e_hip:.3g}")
    bound = atol + rtol * ref64.abs() + slack * e_ref
    bad = err > bound
    assert not bool(bad.any()), (f"{what}: {int(bad.sum())} of {bad.numel()} elements outside rel {rtol} / abs {atol} "
                                 f"+ {slack} x e_ref ({e_ref:.3g}); max |hip - f64| = {e_hip:.3g}")
    return e_ref, e_hip


def assert_parity_of(got, reference, what="", **kw):
    """assert_parity for a kernel whose reference is a formula: reference(dtype) evaluates it on the CPU in that
    dtype (a tensor or a tuple of tensors matching got), once in float32 and once in float64."""
    r32, r64 = reference(torch.float32), reference(torch.float64)
    if isinstance(got, (tuple, list)):
        assert len(got) == len(r32) == len(r64)
        return [assert_parity(g, a, b, f"{what}[{i}]", **kw) for i, (g, a, b) in enumerate(zip(got, r32, r64))]
    return assert_parity(got, r32, r64, what, **kw)
