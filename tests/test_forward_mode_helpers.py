"""Host logic of the forward-mode helpers (learned-dynamics_amd/differentiable.py): add / sub / mul with a tangent on
one side only against torch's own forward-mode rules and against torch.autograd.functional.jvp, on the CPU in float64
(no kernel of the library runs here)."""
import importlib

import torch
import torch.autograd.forward_ad as fwAD


def _diff():
    return importlib.import_module("learned-dynamics_amd.differentiable")


def test_one_sided_arithmetic_equals_torchs_rules():
    diff = _diff()
    torch.manual_seed(0)
    x, u = torch.randn(4, 1, 3, dtype=torch.float64), torch.randn(4, 1, 3, dtype=torch.float64)
    c = torch.randn(5, 3, dtype=torch.float64, requires_grad=True)

    def with_helpers(xx):
        return diff.mul(diff.sub(2.0, diff.add(diff.mul(xx, c), c)), diff.sub(xx, 0.5)) + diff.sub(c, xx) + diff.div(xx, 3.0) \
            + diff.div(xx, c.exp())

    def plain(xx):
        return (2.0 - (xx * c + c)) * (xx - 0.5) + (c - xx) + xx / 3.0 + xx / c.exp()

    assert torch.equal(with_helpers(x), plain(x))                       # outside forward mode: plain arithmetic
    value, tangent = diff.jvp(with_helpers, (x,), (u,))
    value_n, tangent_n = torch.autograd.functional.jvp(plain, (x,), (u,), create_graph=True)
    torch.testing.assert_close(value, value_n, rtol=0, atol=1e-14)
    torch.testing.assert_close(tangent, tangent_n, rtol=0, atol=1e-13)
    g, = torch.autograd.grad((tangent ** 2).sum() + value.sum(), [c])
    g_n, = torch.autograd.grad((tangent_n ** 2).sum() + value_n.sum(), [c])
    torch.testing.assert_close(g, g_n, rtol=0, atol=1e-12)
    with fwAD.dual_level():
        xd = fwAD.make_dual(x, u)
        ours, theirs = fwAD.unpack_dual(with_helpers(xd)), fwAD.unpack_dual(plain(xd))
        torch.testing.assert_close(ours.tangent, theirs.tangent, rtol=0, atol=1e-13)


def test_tangent_detection():
    diff = _diff()
    x = torch.randn(3)
    assert not diff.has_tangent(x) and not diff.has_tangent(None) and not diff.differentiated(x)
    assert diff.differentiated(x.clone().requires_grad_())
    with fwAD.dual_level():
        xd = fwAD.make_dual(x, torch.ones(3))
        assert diff.has_tangent(xd) and diff.differentiated(xd) and not diff.has_tangent(x)
        with torch.no_grad():
            assert diff.differentiated(xd) and diff.wants_grad(torch.nn.Identity(), xd)
    assert not diff.has_tangent(xd)


def test_jvp_of_a_function_without_dependence_gives_zeros():
    diff = _diff()
    value, tangent = diff.jvp(lambda x: torch.ones(2), (torch.randn(2),), (torch.randn(2),))
    assert torch.equal(value, torch.ones(2)) and torch.equal(tangent, torch.zeros(2))


def test_jvp_of_a_function_with_several_results():
    diff = _diff()
    x, u = torch.randn(3, dtype=torch.float64), torch.randn(3, dtype=torch.float64)
    values, tangents = diff.jvp(lambda t: (t.sin(), t * t), (x,), (u,))
    torch.testing.assert_close(values[0], x.sin()); torch.testing.assert_close(values[1], x * x)
    torch.testing.assert_close(tangents[0], x.cos() * u); torch.testing.assert_close(tangents[1], 2 * x * u)


def test_jvp_takes_the_arguments_of_functional_jvp():
    diff = _diff()
    x, u = torch.randn(3, dtype=torch.float64), torch.randn(3, dtype=torch.float64)
    f = lambda t: t.exp() * t
    ours = diff.jvp(f, x, u, create_graph=True)
    theirs = torch.autograd.functional.jvp(f, x, u, create_graph=True)
    torch.testing.assert_close(ours[0], theirs[0]); torch.testing.assert_close(ours[1], theirs[1])
