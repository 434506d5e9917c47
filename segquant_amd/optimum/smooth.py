"""SmoothQuant and SVD (low-rank + residual) optimisers of a segmented linear.

Counterparts of ``SmoothOptimizer`` and ``SVDOptimizer``
(segquant/optimum/optimizer.py:296-575 and :576-731) for what they do at
calibration and at inference:

* ``trace`` records per-input-channel maxima of activations and weights,
  ``smooth`` turns them into the per-channel factors
  ``s = max_x^alpha / max_w^(1 - alpha)`` (:440-457), multiplies the weights by
  ``s`` and -- SVD -- splits each smoothed weight chunk into a rank-``r`` part
  ``L1 L2`` and a residual, which is what gets quantised (:640-684);
* the forward divides the activations by ``s`` and adds ``(x / s) L1 L2`` to
  the quantised product (:514-517, :698-731).

Two routes run the forward.  ``forward`` is the reference's: one ``(S, ...)``
tensor of smoothed inputs through ``call_func``, then two ``bmm`` and an
addition for the low-rank branch.  ``fused_launches`` (input segmentation or a
single chunk) keeps everything inside the two kernels of the fused route: the
division by ``s`` happens in the quantise kernel (``col_div``), every K segment
is a range with its own activation and weight scales, and the low-rank product
is added by the GEMM's epilogue on the matrix cores from ``T = x (L1 / s)``
(M x r, one small library GEMM) and ``L2`` -- the (M, N) product is never
materialised.  With output segmentation every segment smooths the whole input
with its own ``s``, so the reference route (S quantised copies of the input) is
the only one.

The search over ``alpha`` (:519-575) is a calibration-time search outside the
kernel path and is not built: ``search_alpha_config`` with ``enable`` raises.
"""
from __future__ import annotations

import torch

from .. import ops
from .optimizer import BaseOptimizer, DefaultOptimizer, OptimizerRegistry, _as_f32, _FMT


@OptimizerRegistry.register("smooth")
class SmoothOptimizer(DefaultOptimizer):
    def __init__(self, seg_mode, chunks, chunksizes, weight_manager, input_calibrators, weight_calibrators,
                 real_quant=False, dual_scale=False, kernel_type=None, dual_segments=None, alpha=0.5,
                 search_alpha_config=None, verbose=False, **kwargs):
        if seg_mode not in ("input", "weight"):
            raise ValueError("seg_mode not found")
        if len(set(chunksizes)) != 1:
            raise NotImplementedError("Only support equal chunksizes.")
        if len(input_calibrators) != chunks or len(weight_calibrators) != chunks:
            raise AssertionError("smooth / svd optimisers take one input and one weight calibrator per chunk")
        if search_alpha_config is not None and search_alpha_config.get("enable"):
            raise NotImplementedError("the search over alpha is a calibration-time search outside the kernel path")
        BaseOptimizer.__init__(self, seg_mode, chunks, chunksizes, weight_manager, input_calibrators, weight_calibrators,
                               real_quant, dual_scale, kernel_type, dual_segments)
        self.alpha = [alpha] * chunks
        self.max_x, self.max_w = [], []
        self.s = [None] * chunks
        self.has_smoothed = False
        self.has_traced_w = False
        self.search_alpha = False
        self.verbose = verbose

    def __repr__(self):
        head = f"{type(self).__name__}(alpha={self.alpha}" + (f",kernel={self.kernel_type}\n" if self.real_quant else "\n")
        iq = ",\n      ".join(repr(c) for c in self.input_calibrators)
        wq = ",\n      ".join(repr(c) for c in self.weight_calibrators)
        return head + f"    input_quantizers=[\n      {iq}\n  ],\n    weight_quantizers=[\n      {wq}\n  ]\n)"

    # ---- chunk views ------------------------------------------------------
    def _x_chunks(self, x):
        """Per-chunk views of the input: K blocks (input segmentation) or the whole input S times."""
        return list(x.split(self.chunksizes, dim=-1)) if self.seg_mode == "input" else [x] * self.chunks

    def _w_chunks(self):
        """Per-chunk views of the float (out, in) weight: column blocks or row blocks."""
        w = self.weight_manager.weight_tensor
        return list(w.split(self.chunksizes, dim=1 if self.seg_mode == "input" else 0))

    # ---- trace -> smooth (optimizer.py:397-457) ------------------------------
    def trace(self, input_manager):
        x = input_manager.input_tensor
        for i, chunk in enumerate(self._x_chunks(x)):
            m = chunk.abs().reshape(-1, chunk.shape[-1]).amax(dim=0)
            if len(self.max_x) < self.chunks:
                self.max_x.append(m)
            else:
                self.max_x[i] = torch.maximum(self.max_x[i], m)
        if not self.has_traced_w:
            self.max_w = [c.abs().amax(dim=0) for c in self._w_chunks()]
            self.has_traced_w = True

    def smooth(self):
        assert len(self.max_x) == self.chunks and len(self.max_w) == self.chunks, "trace the layer first"
        eps = 1.0 / (1 << 31)
        for i, wc in enumerate(self._w_chunks()):
            s = (self.max_x[i] ** self.alpha[i]) / (self.max_w[i] ** (1 - self.alpha[i]))
            s = torch.where(s <= eps, torch.ones_like(s), s)
            self.s[i] = torch.clamp(s.to(torch.float32), min=1e-4, max=1e4)
            wc.mul_(self.s[i].to(wc.device))
        self.has_smoothed = True
        self._plan = None

    def _smoothed(self, chunk, i):
        """x / s in the input's dtype, as ``input_chunk.div_(s.to(dtype))`` on a clone (:467-470)."""
        return chunk / self.s[i].to(device=chunk.device, dtype=chunk.dtype)

    # ---- calibration ---------------------------------------------------------
    def calibrate(self, input_manager):
        assert self.has_smoothed, "SmoothOptimizer: linear is not smoothed"
        x = input_manager.input_tensor
        chunks = [self._smoothed(c, i) for i, c in enumerate(self._x_chunks(x))]
        for cal, c in zip(self.input_calibrators, chunks):
            cal.calibrate(c)
        for cal, wc, c in zip(self.weight_calibrators, self._w_chunks(), chunks):
            cal.calibrate(wc, input_data=c)

    def finish_calibrate(self):
        for i, cal in enumerate(self.input_calibrators):
            cal.finish_calibrate()
            self.input_calibrators[i] = cal.quantizer
        parts = []
        for i, (cal, wc) in enumerate(zip(self.weight_calibrators, self._w_chunks())):
            parts.append(cal.finish_calibrate(wc.contiguous()).reshape(wc.shape[0], -1))
            self.weight_calibrators[i] = cal.quantizer
        wm = self.weight_manager
        wm.weight_tensor = torch.cat(parts, dim=1 if self.seg_mode == "input" else 0).contiguous()
        wm.packed = self.packed
        self.has_calibrated = True
        self.make_scale_tensor()
        self.max_x = self.max_w = None

    # ---- the reference's route (:514-517) -------------------------------------
    def _smoothed_view(self, input_manager):
        views = input_manager.iter_view()
        return torch.stack([self._smoothed(v, i) for i, v in enumerate(views)])

    def forward(self, input_manager):
        return self.call_func(self._smoothed_view(input_manager), self.weight_manager.iter_view())

    def forward_fake(self, x):
        raise NotImplementedError("smooth / svd layers have equal chunks and take forward()")

    # ---- the fused route --------------------------------------------------------
    def fused_available(self) -> bool:
        one_input = self.seg_mode == "input" or self.chunks == 1
        return bool(self.real_quant and self.has_calibrated and one_input and self.chunks <= ops.L.SEGQ_MAX_KSEG)

    def _build_plan(self, device):
        wm = self.weight_manager
        N, K = wm.out_features, wm.in_features
        fa = _FMT[self.kernel_type.split("A", 1)[1]]
        fw = _FMT[self.kernel_type[1:].split("A", 1)[0]]
        if getattr(self.weight_calibrators[0], "group_size", None) is not None:
            raise NotImplementedError("group-wise weight scales are not combined with smoothing")
        wcodes = wm.weight_tensor.reshape(N, K // 2 if fw == ops.FMT_INT4 else K).contiguous()
        sw_list = [_as_f32(c.scale, device).reshape(-1).contiguous() for c in self.weight_calibrators]
        bounds = [0]
        for c in (self.chunksizes if self.seg_mode == "input" else [K]):
            bounds.append(bounds[-1] + c)
        self._plan = dict(fa=fa, fw=fw, w=wcodes, sw=sw_list[0], sw_list=sw_list, sw_cs=1 if sw_list[0].numel() > 1 else 0,
                          bounds=bounds, N=N, K=K, col_div=torch.cat([s.to(device) for s in self.s]).contiguous())
        return self._plan

    supports_parts = False  # SegmentLinear.forward_parts concatenates and takes forward() instead

    def forward_parts(self, parts, bias=None, pre_ops=None):
        raise NotImplementedError("smooth / svd layers take the concatenated input")


@OptimizerRegistry.register("svd")
class SVDOptimizer(SmoothOptimizer):
    def __init__(self, seg_mode, chunks, chunksizes, weight_manager, input_calibrators, weight_calibrators,
                 real_quant=False, dual_scale=False, kernel_type=None, dual_segments=None, alpha=0.5, low_rank=32,
                 search_alpha_config=None, verbose=False, **kwargs):
        super().__init__(seg_mode, chunks, chunksizes, weight_manager, input_calibrators, weight_calibrators, real_quant,
                         dual_scale, kernel_type, dual_segments, alpha, search_alpha_config, verbose)
        self.low_rank = low_rank
        self.l1s = self.l2s = None
        self.has_svd = False
        self.precision = kwargs.get("precision", "float64")
        if self.precision not in ("float32", "float64"):
            raise ValueError(f"Unsupported precision: {self.precision}. Use 'float32' or 'float64'.")

    def __repr__(self):
        return super().__repr__().replace("(alpha=", f"(low_rank={self.low_rank}, alpha=", 1)

    def _move(self, device):
        super()._move(device)
        if self.l1s is not None:
            self.l1s, self.l2s = self.l1s.to(device), self.l2s.to(device)

    def smooth(self):
        """Smooth, then split every smoothed chunk W_i^T (in, out) into its best rank-r
        approximation ``L1 L2`` (``U_r S_r`` and ``V_r^T`` of the SVD) and the residual, which
        replaces the chunk and is what the calibrators then quantise (:640-684)."""
        super().smooth()
        l1s, l2s = [], []
        for wc in self._w_chunks():
            t = wc.t().to(getattr(torch, self.precision))
            u, sv, vt = torch.linalg.svd(t, full_matrices=False)
            if u.shape[1] < self.low_rank or vt.shape[0] < self.low_rank:
                raise ValueError(f"Low-rank dimension {self.low_rank} exceeds layer dimensions {u.shape[1]} and {vt.shape[0]}.")
            us = u[:, :self.low_rank] * sv[:self.low_rank]
            vt = vt[:self.low_rank, :]
            l1s.append(us.to(device=wc.device, dtype=wc.dtype))
            l2s.append(vt.to(device=wc.device, dtype=wc.dtype))
            wc.copy_((t.to(torch.float64) - (us @ vt).to(torch.float64)).to(dtype=wc.dtype, device=wc.device).t())
        self.l1s = torch.stack(l1s)  # (S, in chunk, r)
        self.l2s = torch.stack(l2s)  # (S, r, out chunk)
        self.has_svd = True

    def calibrate(self, input_manager):
        assert self.has_svd, "SVDOptimizer: linear is not svd"
        super().calibrate(input_manager)

    def _low_rank_mul(self, x, l1s, l2s):
        """(S, ..., k) x (S, k, r) x (S, r, n) with two batched products (:698-722)."""
        lead = x.shape[1:-1]
        x3 = x.reshape(x.shape[0], -1, x.shape[-1])
        out3 = torch.bmm(torch.bmm(x3, l1s.to(x.dtype)), l2s.to(x.dtype))
        return out3.reshape(x.shape[0], *lead, out3.shape[-1])

    def forward(self, input_manager):
        chunks = self._smoothed_view(input_manager)
        return self.call_func(chunks, self.weight_manager.iter_view()) + self._low_rank_mul(chunks, self.l1s, self.l2s)

    def _build_plan(self, device):
        plan = super()._build_plan(device)
        # T = x (L1 / s): the division by s of the reference's (x / s) L1 moved onto the small factor.
        # With input segmentation the S low-rank branches add up: T = [T_1 .. T_S] against the rows of
        # [L2_1; ..; L2_S], i.e. one branch of rank S r.
        l1 = [(self.l1s[i].to(device=device, dtype=torch.float32) / self.s[i].to(device)[:, None]) for i in range(self.chunks)]
        plan["l1s"] = l1                                                        # (k_i, r) each, fp32
        plan["l2t"] = torch.cat([self.l2s[i].to(device=device, dtype=torch.float32) for i in range(self.chunks)], dim=0).t().contiguous()  # (N, S r)
        plan["l12_cast"] = {}
        return plan

    def _lowrank_operands(self, plan, x2):
        """(T, L2T) for the GEMM's epilogue, in the input's dtype."""
        dt = x2.dtype
        cast = plan["l12_cast"].get(dt)
        if cast is None:
            cast = plan["l12_cast"][dt] = ([l.to(dt) for l in plan["l1s"]], plan["l2t"].to(dt).contiguous())
        l1, l2t = cast
        r = self.low_rank
        bounds = plan["bounds"]
        t = torch.empty((x2.shape[0], r * self.chunks), dtype=dt, device=x2.device)
        for i in range(self.chunks):
            torch.matmul(x2[:, bounds[i]:bounds[i + 1]], l1[i], out=t[:, i * r:(i + 1) * r])
        return t, l2t
