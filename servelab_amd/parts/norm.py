"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w in float32; LayerNorm with a gain and
no bias: y = (x - mean) / sqrt(var + eps) * w, var the mean of the squared deviations.

Reference: servelab/attention/triton/paged_attention.py:76-91 and the vector
in tests/test_triton_kernels.py:57-59.  Here the residual add that precedes
every use (servelab/parallel/tp_model.py:131-133) is fused in.
"""
from .base import Norm, ParamSpec


class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, size: int, eps: float, name: str = "weight"):
        self.size = int(size)
        self.eps = float(eps)
        self.name = name

    def param_specs(self):
        return {self.name: ParamSpec((self.size,), init="gain")}

    def load(self, tensors, rt):
        self.rt = rt
        self.weight = rt.vector(tensors(self.name))

    def forward(self, resid, delta, fuse=False):
        return self.rt.ops.add_rmsnorm(resid, delta, self.weight, self.eps, fuse=fuse)

    def forward_rows(self, resid, delta, rows, fuse=False):
        return self.rt.ops.rows_add_rmsnorm(resid, delta, rows, self.weight, self.eps, fuse=fuse)


class LayerNorm(Norm):
    """Layer norm with a gain and no bias, in float32, fused with the residual
    add before it.  ``delta`` may be a tuple of values that are all added (the
    outputs of sublayers that ran side by side).  Its rows are plain normed rows
    (``fuse`` is not taken up)."""
    graph_safe = True

    def __init__(self, size: int, eps: float, name: str = "weight"):
        self.size = int(size)
        self.eps = float(eps)
        self.name = name

    def param_specs(self):
        return {self.name: ParamSpec((self.size,), init="gain")}

    def load(self, tensors, rt):
        self.rt = rt
        self.weight = rt.vector(tensors(self.name))

    def forward(self, resid, delta, fuse=False):
        return self.rt.ops.add_layernorm(resid, delta, self.weight, self.eps)

    def forward_rows(self, resid, delta, rows, fuse=False):
        return self.rt.ops.add_layernorm(resid, delta, self.weight, self.eps, rows=rows)


class PostRMSNorm(RMSNorm):
    """An RMS norm on a sublayer's output instead of its input: the stream takes
    ``mult`` times the normed output, and the sublayers read the stream itself.
    ``forward_post(resid, y)`` adds mult * norm(y) into the float32 stream in
    place and returns the stream's rows in the activation dtype, which is what
    the next sublayer reads (``y`` None: only those rows)."""

    def __init__(self, size: int, eps: float, mult: float = 1.0, name: str = "weight"):
        super().__init__(size, eps, name)
        self.mult = float(mult)

    def forward_post(self, resid, y):
        return self.rt.ops.add_postnorm(resid, y, self.weight, self.eps, self.mult)
