"""RMSNorm (crates/spite-models/src/dense.rs:175-181): y = x * 1/sqrt(mean(x^2) + eps) * w,
sum and scale in fp32, fused with the residual additions that precede it.

``tanh`` ("dynamic tanh"): y = tanh(alpha * x) * w + b with a learned scalar alpha: a squashing of every
element on its own, without any statistic of the row; fp32, fused with the residual additions in the same way."""
from __future__ import annotations

import torch

from .base import Norm, ParamSpec, register
from ..csrc import hipops


@register("norm", "rms")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, env, width: int, eps: float):
        self.width = int(width)
        self.eps = float(eps)
        self.weight = None

    def params(self):
        return {"weight": ParamSpec((self.width,), kind="vector", init="ones")}

    def load(self, tensors):
        self.weight = tensors["weight"]

    def as_increment(self, y, mult: float):
        """This norm as the last step of a sublayer's result y on its way into the stream."""
        from .base import NormedIncrement
        return NormedIncrement(y, self.weight, float(mult), self.eps)

    def can_project(self, proj) -> bool:
        # the kernel keeps the normed row in LDS for the products
        return proj.dtype == torch.float32 and proj.dim() == 2 and proj.shape[1] == self.width \
            and hipops.add_rmsnorm_can_project(self.width)

    def forward(self, h, out, *, d1=None, d2=None, out32=None, rows=None, write_h=True, proj=None, proj_out=None,
                normed=None, second=None):
        """``normed``: a ``NormedIncrement``'s (y, weight, mult, eps), added like d1 and d2 after its own norm.
        ``second`` = (another RMS norm of the same eps, its output): the same rows under that norm's
        weights too, in one pass (a layer with two norms of one stream)."""
        hipops.add_rmsnorm(h, self.weight, self.eps, out=out, out32=out32, d1=d1, d2=d2, rows=rows,
                           n_rows=(rows.numel() if rows is not None else h.shape[0]), write_h=write_h,
                           proj=proj, proj_out=proj_out, normed=normed,
                           w2=second[0].weight if second is not None else None, out2=second[1] if second is not None else None)

    def takes(self, increment) -> bool:
        """Whether ``forward`` adds this normed increment in its own pass (``normed=``)."""
        from .base import NormedIncrement
        return isinstance(increment, NormedIncrement)

    def pairs_with(self, other) -> bool:
        """Whether ``other`` can be this norm's ``second``: the same kind, width and eps."""
        return isinstance(other, RMSNorm) and other.width == self.width and other.eps == self.eps


@register("norm", "tanh")
class TanhNorm(Norm):
    graph_safe = True
    #: ``forward`` adds a normed increment also where it gathers rows and leaves the stream as it is (the model's last norm)
    takes_gathered = True

    def __init__(self, env, width: int):
        self.width = int(width)
        self.weight = self.bias = self.alpha = None

    def params(self):
        return {"weight": ParamSpec((self.width,), kind="vector", init="ones"),
                "bias": ParamSpec((self.width,), kind="vector", init="normal"),
                "alpha": ParamSpec((), kind="vector", init="ones")}

    def load(self, tensors):
        self.weight, self.bias = tensors["weight"].contiguous(), tensors["bias"].contiguous()
        self.alpha = tensors["alpha"].reshape(1).contiguous()

    def as_increment(self, y, mult: float):
        """This norm as the last step of a sublayer's result y on its way into the stream."""
        from .base import TanhIncrement
        return TanhIncrement(y, self.weight, self.bias, self.alpha, float(mult))

    def takes(self, increment) -> bool:
        """Whether ``forward`` adds this normed increment in its own pass (``normed=``)."""
        from .base import TanhIncrement
        return isinstance(increment, TanhIncrement)

    def can_project(self, proj) -> bool:
        # the kernel keeps the normed row in LDS for the products
        return proj.dtype == torch.float32 and proj.dim() == 2 and proj.shape[1] == self.width \
            and hipops.add_tanh_norm_can_project(self.width)

    def forward(self, h, out, *, d1=None, d2=None, out32=None, rows=None, write_h=True, normed=None, plain=False,
                proj=None, proj_out=None):
        """``normed``: a ``TanhIncrement``'s arguments, added like d1 and d2 after its own norm.  ``plain``: out is the
        stream itself (everything added) in out's dtype, not normed.  ``proj`` / ``proj_out``: small fp32 products of
        the normed rows formed in the same pass (router logits)."""
        w, b, a = (None, None, None) if plain else (self.weight, self.bias, self.alpha)
        hipops.add_tanh_norm(h, w, b, a, out=out, out32=out32, d1=d1, d2=d2, rows=rows,
                             n_rows=(rows.numel() if rows is not None else h.shape[0]), write_h=write_h, normed=normed,
                             proj=proj, proj_out=proj_out)
