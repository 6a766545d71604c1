"""Ant16 forward (ant16_o0/o1/o2/oc_cuda and the Ant16 autograd function) against the float64
oracle (oracle/products.py: the einsum forms of managan/codegen_tensor_products.py:112-133), at the
reference's own test shapes (codegen_tensor_products.py:135-140: batch 10, dims 64/48/32, dim_l 16)
and at ragged ones (tile tails, dim_l 8 as in archs/diffuser_atoms5.py:218, channel counts that are
not multiples of 32, a single row, no rows)."""
import importlib

import pytest
import torch

from oracle import products as OP

pytestmark = pytest.mark.gpu


def _inputs(batch, d0, d1, d2, dl, seed):
    g = torch.Generator().manual_seed(seed)
    dims = (d0, d1, d2)
    x = [torch.randn(batch, dims[k], *([3] * k), generator=g) for k in range(3)]
    P = {lab: torch.randn(dims[int(lab[2])], dl, dims[int(lab[1])], generator=g) / (dl * dims[int(lab[1])]) ** 0.5
         for lab in OP.BEE_ORDER}
    left = {lab: torch.randn(batch, dl, *([3] * int(lab[0])), generator=g) for lab in OP.BEE_ORDER}
    return x, P, left


def _args(x, P, left, dev):
    order = ("000", "110", "220", "011", "101", "121", "211", "111", "022", "202", "112", "222", "212")
    flat = [t.to(dev) for t in x]
    for lab in order:                       # argument order of Ant16.forward (codegen_tensor_products.py:21-25)
        flat += [P[lab].to(dev), left[lab].to(dev)]
    return flat


@pytest.mark.parametrize("shape", [(10, 64, 48, 32, 16), (37, 40, 24, 20, 8), (1, 32, 32, 32, 16),
                                   (1000, 64, 48, 32, 16), (65, 130, 7, 33, 5)])
def test_ant16_forward_matches_oracle(shape):
    cg = importlib.import_module("learned-dynamics_amd.codegen_tensor_products")
    batch, d0, d1, d2, dl = shape
    x, P, left = _inputs(batch, d0, d1, d2, dl, seed=sum(shape))
    ref = OP.ant16(*[t.double() for t in x], {k: v.double() for k, v in P.items()},
                   {k: v.double() for k, v in left.items()})
    got = cg.Ant16.apply(*_args(x, P, left, "cuda"))
    for y, r in zip(got, ref):
        assert y.shape == r.shape
        # sums of dim_l * dim_r products of N(0,1) operands per output: rel 1e-5, abs 1e-6 x sqrt(K) x scale
        torch.testing.assert_close(y.cpu().double(), r, rtol=1e-5, atol=1e-6 * float(r.abs().max()) * 4)


def test_ant16_shim_functions_and_errors(ops):
    x, P, left = _inputs(6, 32, 16, 8, 16, seed=5)
    d = lambda t: t.cuda()
    y0, = ops.ant16_o0(d(x[0]), d(x[1]), d(x[2]), d(P["000"]), d(left["000"]), d(P["110"]), d(left["110"]),
                       d(P["220"]), d(left["220"]))
    ref = sum(torch.einsum(OP._ANT_FORMS[lab], left[lab].double(), x[int(lab[1])].double(), P[lab].double())
              for lab in ("000", "110", "220"))
    torch.testing.assert_close(y0.cpu().double(), ref, rtol=1e-5, atol=4e-6 * float(ref.abs().max()))
    y1c, y2c = ops.ant16_oc(d(x[1]), d(x[2]), d(P["111"]), d(left["111"]), d(P["212"]), d(left["212"]))
    assert y1c.shape == (6, 16, 3) and y2c.shape == (6, 8, 3, 3)
    with pytest.raises(RuntimeError, match="P_110: expected axis 2 to have size dim_1"):
        ops.ant16_o0(d(x[0]), d(x[1]), d(x[2]), d(P["000"]), d(left["000"]), d(P["220"]), d(left["110"]),
                     d(P["220"]), d(left["220"]))
    with pytest.raises(RuntimeError, match="x_1 has wrong number of axes"):
        ops.ant16_o0(d(x[0]), d(x[0]), d(x[2]), d(P["000"]), d(left["000"]), d(P["110"]), d(left["110"]),
                     d(P["220"]), d(left["220"]))
    # no rows: empty outputs, nothing launched
    e = [t[:0].cuda() for t in x]
    y0, = ops.ant16_o0(e[0], e[1], e[2], d(P["000"]), d(left["000"][:0]), d(P["110"]), d(left["110"][:0]),
                       d(P["220"]), d(left["220"][:0]))
    assert y0.shape == (0, 32)
