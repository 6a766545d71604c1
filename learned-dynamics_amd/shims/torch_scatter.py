"""Drop-in for the one torch_scatter symbol the reference uses:
segment_coo(src, index, out=None, dim_size=None, reduce="sum")
(call site managan/graph_layers.py:57), for a sorted index along dim 0."""
import importlib

_gl = importlib.import_module("learned-dynamics_amd.graph_layers")


def segment_coo(src, index, out=None, dim_size=None, reduce="sum"):
    if reduce not in ("sum", "add"):
        raise NotImplementedError("only reduce='sum' is implemented")
    if index.dim() != 1:
        raise NotImplementedError("only a 1-D sorted index along dim 0 is implemented")
    if dim_size is None:
        dim_size = int(index[-1].item()) + 1 if index.numel() > 0 else 0
    ans = _gl.segment_sum(src, index, dim_size)
    if out is not None:
        out.copy_(ans)
        return out
    return ans
