"""RMS norm: y = weight * x * rsqrt(mean(x^2) + eps), statistics in float32
(worker/src/inference/qwen2/model.py:77-90). The reference multiplies by the weight
after rounding back to the model dtype; here the product is rounded once."""

from __future__ import annotations

from .base import Norm, ParamSpec, register_part


class RMSNorm(Norm):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.size = int(spec.params["size"])
        self.eps = float(spec.params["eps"])
        self.weight = None

    def param_specs(self):
        return {"weight": ParamSpec((self.size,), "ones")}

    def load(self, tensors) -> None:
        self.weight = tensors["weight"].contiguous()

    def apply(self, ops, x, out_dtype):
        return ops.rmsnorm(x, self.weight, self.eps, out_dtype)

    def add_apply(self, ops, residual, delta, out_dtype):
        return ops.add_rmsnorm(residual, delta, self.weight, self.eps, out_dtype)


register_part("norm", "rmsnorm", RMSNorm)
