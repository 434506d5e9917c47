"""Quantisers: running-amax calibration, scale formulas, fake quantisation and
the hand-off of weights to the code-generating kernels.

Behavioural counterpart of segquant/quantizers/quantizer.py for the symmetric
integer and e4m3 cases the kernel path uses (scale formulas :161-248 and
:398-452, fake quantisation :250-281 and :484-528, weight quantisation
:286-336 and :530-580).  Asymmetric integer quantisation exists in the
reference only on the fake path and is kept here on the fake path too.
"""
from __future__ import annotations

import torch

from ..utils.extension import (load_fake_quant_fp8_ext, load_real_quant_fp8_ext, load_real_quant_int4_ext,
                               load_real_quant_int8_ext)

EPS = 1.0 / (1 << 24)


def _bcast(x: torch.Tensor, s, axis):
    """Reshape a per-axis scale so it broadcasts against ``x`` (the reduced
    axis is re-inserted as size 1)."""
    if not isinstance(s, torch.Tensor) or axis is None:
        return s
    axis = axis if axis >= 0 else x.dim() + axis
    shape = list(s.shape)
    while len(shape) < x.dim():
        shape.insert(axis, 1)
    return s.view(*shape)


class BaseQuantizer:
    def __init__(self, axis=None, dual_scale=False, real_quant=False, dynamic=False, dummy=False, group_size=None):
        # group_size: weights only, with axis=1 -- one scale per (row, run of group_size
        # input channels) instead of one per row.  Not in the reference (its weight scales
        # are per tensor or per row); the scale has shape (rows, in_features / group_size).
        self.group_size = group_size
        if group_size is not None and (axis != 1 or dual_scale or dynamic):
            raise AssertionError("group_size is for static weight scales on axis 1")
        self.axis = axis
        self.dual_scale = dual_scale
        self.real_quant = real_quant
        self.dynamic = dynamic
        self.dummy = dummy
        if real_quant and axis not in (None, 1, -1):
            raise AssertionError("only support axis = -1 for input and axis = 1 for weight")
        self.scale = 1.0
        self.pos_scale = None
        self.neg_scale = None
        self.zero_point = 0
        self.reset()

    # limits of the two signs; subclasses set them
    pos_limit = neg_limit = 1.0

    def reset(self):
        self.amax = self.amin = self.pos_amax = self.neg_amax = None

    def to(self, device):
        for name in ("zero_point", "scale", "pos_scale", "neg_scale", "amax", "amin", "pos_amax", "neg_amax"):
            v = getattr(self, name)
            if isinstance(v, torch.Tensor):
                setattr(self, name, v.to(device))
        return self

    def _track(self, name, value):
        old = getattr(self, name)
        if isinstance(value, torch.Tensor):
            new = value if old is None else torch.maximum(old, value)
        else:
            new = max(old or 0.0, value)
        setattr(self, name, new)
        return new

    @staticmethod
    def _ratio(limit, amax):
        if isinstance(amax, torch.Tensor):
            return limit / amax.clamp(min=EPS)
        return limit / amax if amax > EPS else 1.0

    def _calibrate_symmetric(self, x: torch.Tensor):
        if self.dual_scale:
            if self.axis is None:
                neg, pos = x[x < 0], x[x > 0]
                nmax = neg.abs().max().item() if neg.numel() else 0.0
                pmax = pos.max().item() if pos.numel() else 0.0
            else:
                zero = torch.zeros_like(x)
                nmax = torch.where(x < 0, -x, zero).amax(dim=self.axis)
                pmax = torch.where(x > 0, x, zero).amax(dim=self.axis)
            self.neg_scale = self._ratio(self.neg_limit, self._track("neg_amax", nmax))
            self.pos_scale = self._ratio(self.pos_limit, self._track("pos_amax", pmax))
        else:
            if self.group_size is not None:
                a = self._grouped(x).abs().amax(dim=-1)
            else:
                a = x.abs().max().item() if self.axis is None else x.abs().amax(dim=self.axis)
            self.scale = self._ratio(self.pos_limit, self._track("amax", a))
        self.zero_point = 0

    def _grouped(self, x: torch.Tensor) -> torch.Tensor:
        if x.dim() != 2 or x.shape[1] % self.group_size:
            raise ValueError(f"group_size {self.group_size} needs a 2-D weight whose columns it divides")
        return x.reshape(x.shape[0], x.shape[1] // self.group_size, self.group_size)

    def calibrate(self, x: torch.Tensor):
        if self.dummy:
            self.scale = self.pos_scale = self.neg_scale = 1.0
            self.zero_point = 0
            return
        self._calibrate_symmetric(x)

    def fake_quantize(self, x):
        return self._fake_quantize(x)

    # weights -> codes through the kernels
    def _weight_ext(self):
        raise NotImplementedError

    def quantize(self, x: torch.Tensor) -> torch.Tensor:
        if self.dummy:
            return x
        if self.dynamic:
            self.reset()
            self.calibrate(x)
        if self.real_quant:
            assert not self.dual_scale, "Weight quantization does not support dual scale."
            ext = self._weight_ext()
            if ext is not None and self.group_size is not None:
                g = x.shape[1] // self.group_size
                if not isinstance(self.scale, torch.Tensor) or tuple(self.scale.shape) != (x.shape[0], g):
                    raise ValueError(f"group-wise weight scale must have shape ({x.shape[0]}, {g})")
                scales = self.scale.to(dtype=torch.float32, device=x.device).t().contiguous()
                return ext.quantize_weights_groups(x.contiguous(), scales, self.group_size)
            if ext is not None:
                res = ext.create_quantized_weights(x)
                if self.axis is None:
                    ext.real_quantized_quantize_weights(x.contiguous(), res, float(self.scale))
                else:
                    if self.axis != 1 or not isinstance(self.scale, torch.Tensor) or tuple(self.scale.shape) != (x.shape[0],):
                        raise ValueError(f"per-channel weight scale must have shape ({x.shape[0]},) on axis 1")
                    ext.real_quantized_quantize_weights(
                        x.contiguous(), res, self.scale.to(dtype=torch.float32, device=x.device).contiguous())
                return res
        return self._fake_quantize(x)

    @staticmethod
    def _fmt_amax(t):
        if isinstance(t, torch.Tensor):
            return f"[{t.min().item():.4f}, {t.max().item():.4f}]"
        return "None" if t is None else f"{t:.4f}"


class IntQuantizer(BaseQuantizer):
    def __init__(self, num_bits=8, symmetric=True, axis=None, dual_scale=False, real_quant=False, dynamic=False,
                 dummy=False, group_size=None):
        self.num_bits = num_bits
        self.symmetric = symmetric
        self.qmin = -(2 ** (num_bits - 1))
        self.qmax = 2 ** (num_bits - 1) - 1
        # the negative side has one more code than the positive one
        self.pos_limit = float(self.qmax)
        self.neg_limit = float(-self.qmin)
        if group_size is not None and not symmetric:
            raise AssertionError("group_size is for symmetric weights")
        super().__init__(axis, dual_scale, real_quant, dynamic, dummy, group_size)

    def calibrate(self, x: torch.Tensor):
        if self.dummy or self.symmetric:
            return super().calibrate(x)
        # asymmetric: min/max range mapped onto [qmin, qmax]; fake path only
        if self.axis is None:
            lo, hi = x.min().item(), x.max().item()
            self.amin = lo if self.amin is None else min(self.amin, lo)
            self.amax = hi if self.amax is None else max(self.amax, hi)
            self.scale = (self.qmax - self.qmin) / (self.amax - self.amin)
            self.zero_point = int(round(self.qmin - self.amin * self.scale))
        else:
            lo, hi = x.amin(dim=self.axis), x.amax(dim=self.axis)
            self.amin = lo if self.amin is None else torch.minimum(self.amin, lo)
            self.amax = hi if self.amax is None else torch.maximum(self.amax, hi)
            self.scale = (self.qmax - self.qmin) / (self.amax - self.amin)
            self.zero_point = (self.qmin - self.amin * self.scale).round().to(torch.int)

    def _fake_quantize(self, x: torch.Tensor) -> torch.Tensor:
        if self.symmetric and self.dual_scale:
            ps, ns = _bcast(x, self.pos_scale, self.axis), _bcast(x, self.neg_scale, self.axis)
            nonneg = x >= 0
            q = torch.where(nonneg, torch.clamp(torch.round(x * ps), 0, self.qmax),
                            torch.clamp(torch.round(x * ns), self.qmin, 0))
            return torch.where(nonneg, q / ps, q / ns).to(x.dtype)
        if self.group_size is not None:
            xg, sg = self._grouped(x), self.scale.unsqueeze(-1)
            q = torch.clamp(torch.round(xg * sg), self.qmin, self.qmax)
            return (q / sg).reshape(x.shape).to(x.dtype)
        s = _bcast(x, self.scale, self.axis)
        zp = _bcast(x, self.zero_point, self.axis)
        q = torch.clamp(torch.round(x * s) + zp, self.qmin, self.qmax)
        return ((q - zp) / s).to(x.dtype)

    def _weight_ext(self):
        if self.num_bits == 8:
            return load_real_quant_int8_ext(required=False)[0]
        if self.num_bits == 4:
            return load_real_quant_int4_ext(required=False)[0]
        return None

    def __repr__(self):
        head = (f"IntQuantizer(num_bits={self.num_bits}, symmetric={self.symmetric}, real_quant={self.real_quant}, "
                f"enable={not self.dummy}, dynamic={self.dynamic}, dual_scale={self.dual_scale}, axis={self.axis}, ")
        if self.symmetric and self.dual_scale:
            return head + f"neg_amax={self._fmt_amax(self.neg_amax)}, pos_amax={self._fmt_amax(self.pos_amax)})"
        if self.symmetric:
            return head + f"amax={self._fmt_amax(self.amax)})"
        return head + f"amin={self._fmt_amax(self.amin)}, amax={self._fmt_amax(self.amax)})"


class FloatQuantizer(BaseQuantizer):
    def __init__(self, exp_bits=4, mant_bits=3, axis=None, dual_scale=False, real_quant=False, dynamic=False,
                 dummy=False, group_size=None):
        if group_size is not None:
            raise AssertionError("group_size is for integer weights")
        self.exp_bits = exp_bits
        self.mant_bits = mant_bits
        if (exp_bits, mant_bits) == (4, 3):
            self.fp_max = 448.0
            # smallest value the no-subnormal simulation keeps (reference quantizer.py:384)
            self.fp_min = (2 ** -6) * (240 / 448.0)
        else:
            self.fp_max = (2 ** (2 ** exp_bits - 2)) * (2 - 2 ** (-mant_bits))
            self.fp_min = 2 ** (1 - (2 ** (exp_bits - 1)))
        self.pos_limit = self.neg_limit = self.fp_max
        super().__init__(axis, dual_scale, real_quant, dynamic, dummy)
        self.scale = None

    @staticmethod
    def _simulate_fp(x, fp_min, fp_max, mant_bits):
        """Round to a float grid WITHOUT subnormals: magnitudes below ``fp_min``
        become zero (reference quantizer.py:462-482)."""
        mag = x.abs().clamp(max=fp_max)
        mag = torch.where(mag < fp_min, torch.zeros_like(mag), mag)
        expo = torch.floor(torch.log2(mag.clamp(min=fp_min)))
        frac = torch.round((mag / 2 ** expo - 1) * 2 ** mant_bits) / 2 ** mant_bits
        return (1 + frac) * 2 ** expo * x.sign()

    def _round_trip(self, v):
        if (self.exp_bits, self.mant_bits) == (4, 3):
            ext = load_fake_quant_fp8_ext(required=False)
            if ext is not None:
                return ext.fake_e4m3fy(v)
        return self._simulate_fp(v, self.fp_min, self.fp_max, self.mant_bits)

    def _fake_quantize(self, x: torch.Tensor) -> torch.Tensor:
        tiny = x.abs() < EPS
        if self.dual_scale:
            ps, ns = _bcast(x, self.pos_scale, self.axis), _bcast(x, self.neg_scale, self.axis)
            nonneg = x >= 0
            q = self._round_trip(torch.where(nonneg, x * ps, x * ns))
            out = torch.where(nonneg, q / ps, q / ns)
        else:
            s = _bcast(x, self.scale, self.axis)
            out = self._round_trip(x * s) / s
        out = out.masked_fill(tiny, 0.0)
        return out.to(x.dtype)

    def _weight_ext(self):
        return load_real_quant_fp8_ext(required=False)[0]

    def __repr__(self):
        head = (f"FloatQuantizer(exp_bits={self.exp_bits}, mant_bits={self.mant_bits}, real_quant={self.real_quant}, "
                f"enable={not self.dummy}, dynamic={self.dynamic}, axis={self.axis}, dual_scale={self.dual_scale}, ")
        if self.dual_scale:
            return head + f"neg_amax={self._fmt_amax(self.neg_amax)}, pos_amax={self._fmt_amax(self.pos_amax)})"
        return head + f"amax={self._fmt_amax(self.amax)})"


class QuantizerRegistry:
    """Name -> factory, keyed by ``DType.value`` (reference quantizer.py:83-129, :596-627)."""
    _registry = {}

    @classmethod
    def register(cls, name):
        def wrap(factory):
            cls._registry[name] = factory
            return factory
        return wrap

    @classmethod
    def get(cls, name):
        return cls._registry.get(name)

    @classmethod
    def create(cls, name, **kwargs):
        factory = cls.get(name)
        if factory is None:
            raise ValueError(f"Quantizer '{name}' not found in registry.")
        return factory(**kwargs)


QuantizerRegistry.register("int8")(IntQuantizer)
QuantizerRegistry.register("fpe4m3")(FloatQuantizer)
for _bits in (16, 6, 4):
    QuantizerRegistry.register(f"int{_bits}")(lambda _b=_bits, **kw: IntQuantizer(num_bits=_b, **kw))
QuantizerRegistry.register("fpe5m2")(lambda **kw: FloatQuantizer(exp_bits=5, mant_bits=2, **kw))
QuantizerRegistry.register("fp16")(lambda **kw: FloatQuantizer(exp_bits=5, mant_bits=10, dummy=True, **kw))
QuantizerRegistry.register("bf16")(lambda **kw: FloatQuantizer(exp_bits=8, mant_bits=7, dummy=True, **kw))
