"""The part of managan/layers_common.py that lies on the path: ScalGroupNorm (managan/layers_common.py:201-223), under
the reference's module name."""
from .painn import ScalGroupNorm

__all__ = ["ScalGroupNorm"]
