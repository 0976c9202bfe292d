"""RMSNorm.  Formula of engine/kernels/triton/rmsnorm.py:19-42 (float32 sum of
squares, rstd = rsqrt(sum/dim + eps), x*rstd*w, one rounding at the store)."""

from __future__ import annotations

from tokensprint_amd.parts.base import NORMS, Norm, TensorDecl, register


@register(NORMS, "rmsnorm")
class RMSNorm(Norm):
    """params: dim, eps, weight (checkpoint name), one_plus (the checkpoint stores the weight
    around zero and the norm multiplies by 1 + w; the sum is made once, when the weight is
    loaded, in float32), scalar (the checkpoint holds one number for all coordinates; it is
    spread over `dim` values when it is loaded, so every fused form of the norm serves it)."""

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        self.dim = int(params["dim"])
        self.eps = float(params["eps"])
        self.weight_name = params["weight"]
        self.one_plus = bool(params.get("one_plus", False))
        self.scalar = bool(params.get("scalar", False))
        self.weight = None

    def tensors(self):
        return {self.weight_name: TensorDecl(() if self.scalar else (self.dim,), role="vector",
                                             init=(-0.3, 0.3) if self.one_plus else None)}

    def load(self, get):
        self.weight = get(self.weight_name)
        if self.scalar:
            self.weight = self.weight.float().reshape(1).expand(self.dim).contiguous()
        if self.one_plus:
            self.weight = (self.weight.float() + 1.0).contiguous()

    def fused_rmsnorm(self):
        return self.weight, self.eps

    def forward(self, x):
        return self.ops.rmsnorm(x, self.weight, self.eps, self.ctx.dtype)

    def add_forward(self, resid, delta):
        return self.ops.add_rmsnorm(resid, delta, self.weight, self.eps, self.ctx.dtype)
