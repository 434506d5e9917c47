"""The optimiser owns the quantised weights and scales of one segmented linear
and is the single call site of the kernels.

Counterpart of ``BaseOptimizer`` / ``DefaultOptimizer``
(segquant/optimum/optimizer.py:10-123, :147-293).  Two routes reach the GPU:

* :meth:`BaseOptimizer.call_func` keeps the reference's call
  ``ext_dict[kernel_type][func_name](X, W, scales...)`` on ``(S, ...)`` tensors
  and returns per-segment outputs.
* :meth:`DefaultOptimizer.forward_fused` is this build's own route: one
  quantise launch and one GEMM launch on the un-replicated input, segments
  expressed as a per-column scale vector (weight-seg) or K ranges (input-seg),
  bias added in the epilogue, output already in its final layout.

The smoothing and low-rank optimisers of the reference are calibration-time
algebra outside the kernel path and are not built.
"""
from __future__ import annotations

import torch

from .. import ops
from ..layers import ext_dict
from ..layers.segment_tensor_manager import InputSegmentTensorManager, segmented_matmul

_FMT = {"int8": ops.FMT_INT8, "int4": ops.FMT_INT4, "fpe4m3": ops.FMT_E4M3}


def _as_f32(v, device):
    if isinstance(v, torch.Tensor):
        return v.to(dtype=torch.float32, device=device)
    return torch.tensor(v, dtype=torch.float32, device=device)


class BaseOptimizer:
    def __init__(self, seg_mode, chunks, chunksizes, weight_manager, input_calibrators, weight_calibrators,
                 real_quant=False, dual_scale=False, kernel_type=None, dual_segments=None):
        self.seg_mode = seg_mode
        self.chunks = chunks
        self.chunksizes = chunksizes
        self.weight_manager = weight_manager
        self.input_calibrators = input_calibrators
        self.weight_calibrators = weight_calibrators
        self.real_quant = real_quant
        self.kernel_type = kernel_type
        self.packed = bool(real_quant and "Wint4" in (kernel_type or ""))
        self.dual_scale = dual_scale
        # which input calibrators are DualScale (this build allows a mix: e.g. the
        # attention half of a concatenated input single-scale, the MLP half dual)
        self.dual_segments = list(dual_segments) if dual_segments is not None else [dual_scale] * len(input_calibrators)
        self.func_name = "gemm_dual_scaled_fn" if (real_quant and dual_scale) else "gemm_scaled_fn"
        self.has_calibrated = False
        self.scale_tensor = None
        self._plan = None

    def _stack(self, calibrators, attr):
        dev = self.weight_manager.device()

        def pick(c):
            v = getattr(c, attr)
            # a single-scale quantiser in a DualScale layer uses its one scale for both signs
            return c.scale if v is None and attr in ("pos_scale", "neg_scale") else v

        vals = [_as_f32(pick(c), dev) for c in calibrators]
        if len(vals) == 1:
            vals = vals * self.chunks
        if len({tuple(v.shape) for v in vals}) != 1:
            return None  # unequal segments: only the fused route and the fake path apply
        return torch.stack(vals)

    def make_scale_tensor(self):
        """(S,) or (S, M) input scales and (S,) or (S, n) weight scales, fp32 on
        the weight's device; DualScale gives (pos, neg, weight)."""
        w = self._stack(self.weight_calibrators, "scale")
        if self.dual_scale:
            self.scale_tensor = (self._stack(self.input_calibrators, "pos_scale"),
                                 self._stack(self.input_calibrators, "neg_scale"), w)
        else:
            self.scale_tensor = (self._stack(self.input_calibrators, "scale"), w)
        self._plan = None

    def call_func(self, batch_input: torch.Tensor, batch_weight: torch.Tensor):
        if self.real_quant:
            if getattr(self.weight_calibrators[0], "group_size", None) is not None:
                # the reference's operators take one weight scale per segment or per row
                raise NotImplementedError("group-wise weight scales run on the fused route only (chunked=False)")
            if self.input_calibrators[0].dynamic:
                # The reference calls a method that does not exist here
                # (optimizer.py:96-100).  Recalibrate each segment on this
                # input instead; the fused route does this inside the kernel.
                for cal, chunk in zip(self.input_calibrators, batch_input):
                    cal.reset()
                    cal.calibrate(chunk)
                self.make_scale_tensor()
            fn = ext_dict[self.kernel_type][self.func_name]
            args = [t.contiguous() for t in self.scale_tensor]
            return fn(batch_input.contiguous(), batch_weight.contiguous(), *args)
        # fake path: quantise-dequantise each segment, then a float matmul.
        # The input is not modified (the reference writes into a view of it).
        quantised = torch.stack([self.input_calibrators[min(i, len(self.input_calibrators) - 1)].quantize(seg)
                                 for i, seg in enumerate(batch_input)])
        return segmented_matmul(quantised, batch_weight)

    def process_step(self, err):
        pass

    def to_cpu(self):
        self._move("cpu")

    def to_cuda(self, device):
        self._move(device)

    def _move(self, device):
        self.weight_manager = self.weight_manager.to(device)
        self.input_calibrators = [c.to(device) for c in self.input_calibrators]
        self.weight_calibrators = [c.to(device) for c in self.weight_calibrators]
        if self.scale_tensor is not None:
            self.scale_tensor = tuple(t.to(device) if t is not None else None for t in self.scale_tensor)
        self._plan = None


class OptimizerRegistry:
    _registry = {}

    @classmethod
    def register(cls, name):
        def wrap(c):
            cls._registry[name] = c
            return c
        return wrap

    @classmethod
    def get(cls, name):
        return cls._registry.get(name)

    @classmethod
    def create(cls, name, **kwargs):
        c = cls.get(name)
        if c is None:
            raise ValueError(f"Optimizer '{name}' not found in registry.")
        return c(**kwargs)


_MAX_CACHED_TOKEN_COUNTS = 8  # (token count, dtype, bias) entries a layer keeps launch descriptors and buffers for


@OptimizerRegistry.register("default")
class DefaultOptimizer(BaseOptimizer):
    def __init__(self, seg_mode, chunks, chunksizes, weight_manager, input_calibrators, weight_calibrators,
                 real_quant=False, dual_scale=False, kernel_type=None, dual_segments=None, **kwargs):
        assert len(input_calibrators) == 1 or len(weight_calibrators) == 1, \
            "Either input_calibrators or weight_calibrators must have a length of 1."
        if seg_mode not in ("input", "weight"):
            raise ValueError("seg_mode not found")
        super().__init__(seg_mode, chunks, chunksizes, weight_manager, input_calibrators, weight_calibrators,
                         real_quant, dual_scale, kernel_type, dual_segments)

    def __repr__(self):
        head = f"DefaultOptimizer(type={self.kernel_type}\n" if self.real_quant else "DefaultOptimizer(\n"
        iq = ",\n    ".join(repr(c) for c in self.input_calibrators)
        wq = ",\n    ".join(repr(c) for c in self.weight_calibrators)
        return head + f"    input_quantizers=[\n    {iq}\n  ],\n    weight_quantizers=[\n    {wq}\n  ]\n)"

    def _input_segments(self, x):
        """The tensor each input calibrator sees: column blocks for input
        segmentation (sizes may differ), the whole input otherwise."""
        if self.seg_mode == "input":
            return x.split(self.chunksizes, dim=-1)
        return [x]

    def calibrate(self, input_manager: InputSegmentTensorManager):
        x = input_manager.input_tensor
        for cal, chunk in zip(self.input_calibrators, self._input_segments(x)):
            cal.calibrate(chunk)
        w = self.weight_manager.weight_tensor
        # input-seg: one weight calibrator sees the whole matrix; weight-seg: one per row block
        blocks = [w] if self.seg_mode == "input" else w.split(self.chunksizes, dim=0)
        for cal, wb in zip(self.weight_calibrators, blocks):
            cal.calibrate(wb, input_data=x)

    def finish_calibrate(self):
        for i, cal in enumerate(self.input_calibrators):
            cal.finish_calibrate()
            self.input_calibrators[i] = cal.quantizer
        wm = self.weight_manager
        w = wm.weight_tensor
        blocks = [w] if self.seg_mode == "input" else w.split(self.chunksizes, dim=0)
        parts = []
        for i, (cal, wb) in enumerate(zip(self.weight_calibrators, blocks)):
            parts.append(cal.finish_calibrate(wb.contiguous()).reshape(wb.shape[0], -1))
            self.weight_calibrators[i] = cal.quantizer
        # codes (or fake-quantised floats) stay in the (out, in) layout; packed
        # int4 is (out, in/2) bytes, so K segments are byte ranges of each row
        wm.weight_tensor = torch.cat(parts, dim=0) if len(parts) > 1 else parts[0]
        wm.packed = self.packed
        self.has_calibrated = True
        self.make_scale_tensor()

    def forward(self, input_manager: InputSegmentTensorManager):
        """Per-segment outputs (S, ..., n) through the reference-convention
        operator; needs equal segment sizes, as the reference does."""
        if len(set(self.chunksizes)) != 1:
            raise NotImplementedError("Only support equal chunksizes.")
        return self.call_func(input_manager.iter_view(), self.weight_manager.iter_view())

    def forward_fake(self, x: torch.Tensor) -> torch.Tensor:
        """Fake-quantised linear without bias for any segment sizes: quantise-
        dequantise each input block with its own scale, one float matmul."""
        cals = self.input_calibrators
        xq = torch.cat([c.quantize(seg) for c, seg in zip(cals, self._input_segments(x))], dim=-1)
        return xq @ self.weight_manager.weight_tensor.to(xq.dtype).transpose(-1, -2)

    # ---- the fused route -------------------------------------------------
    def fused_available(self) -> bool:
        """The one-launch route serves up to SEGQ_MAX_KSEG input segments; layers with more
        (the reference accepts any number of equal chunks) take the reference-convention
        operator, one batched launch over the segments."""
        few = self.seg_mode != "input" or self.chunks <= ops.L.SEGQ_MAX_KSEG
        return bool(self.real_quant and self.has_calibrated and few)

    def _build_plan(self, device):
        """Turns segments and calibrated scales into what the kernels take."""
        wm = self.weight_manager
        N, K = wm.out_features, wm.in_features
        S = self.chunks
        fa = _FMT[self.kernel_type.split("A", 1)[1]]
        fw = _FMT[self.kernel_type[1:].split("A", 1)[0]]
        wcodes = wm.weight_tensor
        wcodes = wcodes.reshape(N, K // 2 if fw == ops.FMT_INT4 else K).contiguous()
        dev = wm.device()
        group = getattr(self.weight_calibrators[0], "group_size", None)
        if group is not None:
            # group-wise weight scales (rows, K / group): the kernel takes their reciprocals as a
            # (K / group, N) matrix of factors; the per-column scale it also applies is 1
            if group != 128:
                raise NotImplementedError("the kernel path has group-wise weight scales for groups of 128")
            per_row = torch.cat([_as_f32(c.scale, dev).reshape(-1, K // group) for c in self.weight_calibrators])
            bounds = [0, K]
            if self.seg_mode != "weight":
                bounds = [0]
                for c in self.chunksizes:
                    bounds.append(bounds[-1] + c)
            self._plan = dict(fa=fa, fw=fw, w=wcodes, sw=torch.ones(1, dtype=torch.float32, device=device), sw_cs=0,
                              bounds=bounds, N=N, K=K, group_dequant=(1.0 / per_row).t().contiguous().to(device))
            return self._plan
        wscales = [_as_f32(c.scale, dev).reshape(-1) for c in self.weight_calibrators]
        if self.seg_mode == "weight":
            # per-segment or per-channel -> one scale per output column (or a single scalar)
            if S == 1:
                sw_vec = wscales[0]
            else:
                sw_vec = torch.cat([w.expand(n) if w.numel() == 1 else w for w, n in zip(wscales, self.chunksizes)])
            bounds = [0, K]
        else:
            sw_vec = wscales[0]  # one calibrator for the whole matrix
            bounds = [0]
            for c in self.chunksizes:
                bounds.append(bounds[-1] + c)
        self._plan = dict(fa=fa, fw=fw, w=wcodes, sw=sw_vec.contiguous().to(device),
                          sw_cs=1 if sw_vec.numel() > 1 else 0, bounds=bounds, N=N, K=K)
        return self._plan

    def forward_fused(self, x: torch.Tensor, bias=None, pre_op=None, gate=None, col_div=None, addend=None) -> torch.Tensor:
        """Final (..., out) result in ``x.dtype``: the two launches of :meth:`fused_launches`
        through one call of the library (``segq_linear``), or through two when a
        ``record_launches`` block is timing the kernels apart."""
        q, g, ws = self.fused_launches(x, bias, pre_op=pre_op, gate=gate, col_div=col_div, addend=addend)
        if ops.recording_launches():
            ops.quantize_launch(q)
            out = ops.gemm_launch(g, ws)
        else:
            out = ops.linear(q, g, ws)
        return out.view(*x.shape[:-1], out.shape[-1])

    def fused_launches(self, x: torch.Tensor, bias=None, pre_op=None, gate=None, col_div=None, addend=None, fresh=False,
                       out_codes=None):
        """What the fused route enqueues for ``x``, not yet launched: the quantise launch
        (``ops.quantize_desc``), the GEMM that reads its codes (``ops.gemm_desc``, output
        (M, out) in ``x.dtype``) and the workspace this layer lends it (or None).  Callers that
        schedule the two themselves (the quantise step of the next layer under this layer's
        GEMM, say) use ``ops.quantize_launch`` / ``ops.gemm_launch`` on them.  Calls with a token
        count seen before reuse the code and scale tensors of the previous call on the same
        stream (launches on one stream run in order, and the codes only live from the quantise
        launch to the GEMM that follows it); ``fresh=True`` allocates new ones, for callers that
        hold several launches of one layer at once.

        Quantise + segmented GEMM with
        de-quantisation and bias fused.  Equivalent to ``forward`` followed by
        the recombination of ``SegmentLinear.forward``, with the partial sums of
        input segments combined in fp32 and rounded once.

        ``pre_op`` / ``gate``: the layer's input is op(x), or x * op(gate), with
        the activation function evaluated inside the quantise kernel (see
        ``ops.quantize``); the scales must have been calibrated on that input.
        ``col_div``: one divisor per input channel applied before quantising (the
        reference's SmoothQuant step ``x / s``, optimizer.py:467-470; the weights must
        have been multiplied by ``s``).  ``addend``: a (..., out) tensor of ``x.dtype``
        added to the result before its one rounding (the SVD optimiser's low-rank
        branch, optimizer.py:731-740)."""
        plan = self._plan or self._build_plan(x.device)
        K, N = plan["K"], plan["N"]
        x2 = x.reshape(-1, K)
        if not x2.is_contiguous():
            x2 = x2.contiguous()
        if col_div is not None and plan.get("col_div") is not None:
            raise RuntimeError("this layer already divides by its own smoothing factors: an external col_div is not combined with them")
        if col_div is None:
            col_div = plan.get("col_div")  # a smoothed layer's own divisors
        if "l2t" in plan and (pre_op is not None or gate is not None):
            # the low-rank operand T = x (L1 / s) is built from the tensor handed in here, so that
            # tensor must be the layer's input itself, not what is in front of its activation function
            raise RuntimeError("a layer with a low-rank branch takes its activated input: apply pre_op / gate before the call")
        plain = pre_op is None and gate is None and col_div is None and addend is None and "l2t" not in plan and out_codes is None
        if plain:
            hit = plan.setdefault("launches", {}).get((x2.shape[0], x.dtype, None if bias is None else bias.data_ptr()))
            if hit is not None:
                return self._relaunch(hit, x2, fresh)
        if gate is not None:
            gate = gate.reshape(-1, K)
            if not gate.is_contiguous():
                gate = gate.contiguous()
        M = x2.shape[0]
        S = self.chunks if self.seg_mode == "input" else 1
        bounds = plan["bounds"]
        dyn = bool(self.input_calibrators[0].dynamic)
        dual = self.dual_scale
        if dyn:
            if self.input_calibrators[0].axis is None:
                raise NotImplementedError("dynamic activation scales are per token (axis=-1) on the kernel path")
            pos = torch.empty((S, M), dtype=torch.float32, device=x.device)
            neg = torch.empty_like(pos) if dual else None
            per_tok = True
        else:
            pos, neg = self._static_sx(plan, x.device)  # (S, 1) per segment or (S, M) per token
            per_tok = pos.shape[-1] > 1
            if per_tok and pos.shape[-1] != M:
                raise RuntimeError(f"static per-token scales were calibrated for {pos.shape[-1]} tokens, got {M}")
        kstride = M if per_tok else 1
        mask = sum(1 << i for i, d in enumerate(self.dual_segments) if d)
        # DualScale: two code tensors (Xp, Xn).  Reading plain codes lets both
        # operands stream straight into LDS; the single merged tensor would save a
        # third of the quantise traffic but costs the GEMM ~50 % (sign selection in
        # registers), measured on the 4608 x 15360 x 3072 shape.
        q = ops.quantize_desc(x2, plan["fa"], pos, neg, row_stride=1 if per_tok else 0,
                              kseg_bounds=bounds if S > 1 else None, kseg_stride=kstride, dual=dual,
                              dual_kseg_mask=mask, dynamic=dyn, two_tensors=dual, pre_op=pre_op, gate=gate,
                              col_div=col_div)
        codes, codes_neg = q[1] if dual else (q[1], None)
        ranges = []
        for s in range(S):
            k0, k1 = bounds[s], bounds[s + 1]
            rs = 1 if per_tok else 0
            sw_s = plan["sw_list"][s] if "sw_list" in plan else plan["sw"]  # smoothed layers: one weight scale per K segment
            ranges.append(ops.Range(k0, k1 - k0, pos[s], sw_s, 0, rs, plan["sw_cs"]))
            if dual and self.dual_segments[s]:
                ranges.append(ops.Range(k0, k1 - k0, neg[s], sw_s, 1, rs, plan["sw_cs"]))
        ldb = K // 2 if plan["fw"] == ops.FMT_INT4 else K
        gdq = plan.get("group_dequant")
        add2 = None if addend is None else addend.reshape(M, N).contiguous()
        kw = dict(m=M, n=N, a_fmt=plan["fa"], b_fmt=plan["fw"], out_dtype=x.dtype, lda=K, ldb=ldb, bias=bias, a_neg=codes_neg,
                  group_dequant=gdq, out_codes=out_codes)
        g = None
        if "l2t" in plan:
            # the SVD optimiser's low-rank branch: inside the GEMM's epilogue where the library has a
            # kernel for it (16-bit dtypes, the 8-wave kernels), as a materialised (M, N) addend otherwise
            t_lr, l2t = self._lowrank_operands(plan, x2)
            ok = plan.setdefault("lr_ok", {}).get((M, x.dtype))
            if ok is None or ok:
                try:
                    g = ops.gemm_desc(codes, plan["w"], ranges, addend=add2, lowrank=(t_lr, l2t), **kw)
                    if ok is None:
                        ops.gemm_plan(g)
                except RuntimeError:
                    g = None
                plan["lr_ok"][(M, x.dtype)] = g is not None
            if g is None:
                low = t_lr @ l2t.t()
                add2 = low if add2 is None else add2 + low
        if g is None:
            g = ops.gemm_desc(codes, plan["w"], ranges, addend=add2, **kw)
        # Whether to lend the library a workspace is this layer's call; how much it could use is
        # the library's (segq_gemm_workspace_bytes), asked once per token count.
        #  * int4 weights and many tokens: the GEMM is bound by the matrix cores, so the weights are
        #    expanded to int8 once per launch and the int8 kernels run; with few tokens reading half
        #    the weight bytes matters more (measured, K 1280, N 10240: 161 -> 119 us at 8192 tokens,
        #    no gain at 2048).  Group-wise scales run on the int8 kernels only: always lend.
        #  * 8-bit weights: always.  int8 with several ranges (K segments, DualScale) parks the
        #    finished ranges' sums there and keeps the big tiles (4608 x 15360 x 3072, three ranges:
        #    441 -> 383 us; 9216 tokens: 1044 -> 756 us); few tiles and a long K share the K steps of
        #    a tile between workgroups (1024 x 15360 x 3072: 162 -> 108 us int8, 135 -> 98 us e4m3).
        int4 = plan["fw"] == ops.FMT_INT4
        lend = (M >= 3072 or gdq is not None) if int4 else True
        ws = None
        if lend:
            need = plan.setdefault("ws_need", {}).get(M)
            if need is None:
                need = plan["ws_need"][M] = ops.gemm_workspace_bytes(g)
            if need:
                ws = ops.int4_workspace(x.device, need)
        if plain:
            # the same descriptors serve every later call with this token count: only the
            # addresses of what is allocated per call change (see _relaunch)
            sx_src = []
            for s_ in range(S):
                sx_src.append((0, s_))
                if dual and self.dual_segments[s_]:
                    sx_src.append((1, s_))
            # a bounded cache: layers fed with ever-changing token counts would otherwise keep descriptors,
            # code and scale buffers of every count they have seen.  The oldest entry goes (its buffers
            # with it) unless a stream capture is under way, whose graph may hold their addresses
            cache = plan["launches"]
            if len(cache) >= _MAX_CACHED_TOKEN_COUNTS and not torch.cuda.is_current_stream_capturing():
                cache.pop(next(iter(cache)))
            cache[(M, x.dtype, None if bias is None else bias.data_ptr())] = dict(
                q=(q[0], q[2]), g=(g[0], g[2]), need=0 if ws is None else need, dyn=dyn, dual=dual, S=S, M=M, N=N, sx_src=sx_src,
                code_shape=tuple(codes.shape), code_dtype=codes.dtype, out_dtype=x.dtype, static=(pos, neg, bias))
        return q, g, ws

    # ---- chained linears: this layer's GEMM writes the next layer's codes ----------------------
    def accepts_codes(self) -> bool:
        """Whether another layer's GEMM can write this layer's activation codes: static per-tensor
        activation scales (DualScale or not), one K range, no smoothing division or low-rank branch
        (both act on the float input)."""
        if not self.fused_available():
            return False
        cal = self.input_calibrators[0]
        one_range = self.seg_mode != "input" or self.chunks == 1
        plain = getattr(self, "s", None) is None and getattr(self, "l1s", None) is None
        fa = _FMT[self.kernel_type.split("A", 1)[1]]
        return bool(one_range and plain and not cal.dynamic and cal.axis is None and fa in (ops.FMT_INT8, ops.FMT_E4M3))

    def code_spec(self, device, pre_op=None) -> dict:
        """What a producing GEMM needs to write this layer's codes (``ops.gemm_desc(out_codes=...)``)."""
        plan = self._plan or self._build_plan(device)
        pos, neg = self._static_sx(plan, device)
        return dict(fmt=plan["fa"], scale=pos[0], scale_neg=neg[0] if self.dual_scale else None, pre_op=pre_op)

    def writes_codes(self, x: torch.Tensor) -> bool:
        """Whether this layer's GEMM has the epilogue that writes codes for ``x``: plain 8-bit codes on
        both sides, one K range in whole 128-byte steps, a 16-bit input dtype, nothing but the bias
        joining the result."""
        if not self.fused_available() or x.dtype not in (torch.bfloat16, torch.float16):
            return False
        plan = self._plan or self._build_plan(x.device)
        one_range = (self.seg_mode != "input" or self.chunks == 1) and not self.dual_scale
        return bool(one_range and plan["fw"] != ops.FMT_INT4 and plan["fa"] != ops.FMT_INT4 and plan["K"] % 128 == 0 and
                    plan.get("group_dequant") is None and plan.get("col_div") is None and "l2t" not in plan)

    def forward_codes(self, codes, lead_shape, out_dtype, bias=None) -> torch.Tensor:
        """This layer's GEMM on activation codes another launch has written (one tensor, or the
        DualScale pair): the second half of :meth:`forward_fused`."""
        codes, codes_neg = codes if isinstance(codes, tuple) else (codes, None)
        plan = self._plan or self._build_plan(codes.device)
        K, N = plan["K"], plan["N"]
        M = codes.shape[0]
        pos, neg = self._static_sx(plan, codes.device)
        ranges = [ops.Range(0, K, pos[0], plan["sw"], 0, 0, plan["sw_cs"])]
        if self.dual_scale:
            ranges.append(ops.Range(0, K, neg[0], plan["sw"], 1, 0, plan["sw_cs"]))
        g = ops.gemm_desc(codes, plan["w"], ranges, m=M, n=N, a_fmt=plan["fa"], b_fmt=plan["fw"], out_dtype=out_dtype, lda=K,
                          ldb=K // 2 if plan["fw"] == ops.FMT_INT4 else K, bias=bias, a_neg=codes_neg,
                          group_dequant=plan.get("group_dequant"))
        ws = None
        int4 = plan["fw"] == ops.FMT_INT4
        if M >= 3072 or not int4 or plan.get("group_dequant") is not None:
            need = plan.setdefault("ws_need", {}).get(M)
            if need is None:
                need = plan["ws_need"][M] = ops.gemm_workspace_bytes(g)
            if need:
                ws = ops.int4_workspace(codes.device, need)
        out = ops.gemm_launch(g, ws)
        return out.view(*lead_shape, N)

    def _static_sx(self, plan, device):
        """Calibrated activation scales stacked over the input segments: (pos, neg) for DualScale
        layers (a single-scale segment's one scale stands on both sides), (scale, None) otherwise."""
        if "sx" not in plan:
            def stack(attr):
                vals = []
                for c, d in zip(self.input_calibrators, self.dual_segments):
                    vals.append(_as_f32(getattr(c, attr if d else "scale"), device).reshape(-1))
                return torch.stack(vals)
            plan["sx"] = (stack("pos_scale"), stack("neg_scale")) if self.dual_scale else (stack("scale"), None)
        return plan["sx"]

    def forward_parts(self, parts, bias=None, pre_ops=None) -> torch.Tensor:
        """The fused route for a layer whose input is a concatenation, fed by the producers of the
        parts instead of by the concatenated tensor: part s (M, chunksizes[s]) is quantised straight
        into columns [k_s, k_s+1) of the one code tensor the GEMM reads, with the activation
        function ``pre_ops[s]`` of its producer evaluated inside the quantise kernel.  Neither the
        activated part nor the concatenation is ever written to memory (the reference builds both
        with torch operators before the linear, backend/torch/modules/transformer_flux.py:91-101:
        ``torch.cat([attn_output, self.act_mlp(mlp_hidden_states)], dim=2)`` -> ``proj_out``).
        One quantise launch per part, then the GEMM of :meth:`fused_launches`."""
        if self.seg_mode != "input" or len(parts) != self.chunks:
            raise RuntimeError(f"forward_parts takes one tensor per input segment ({self.chunks} of them)")
        pre_ops = list(pre_ops) if pre_ops is not None else [None] * len(parts)
        plan = self._plan or self._build_plan(parts[0].device)
        if plan.get("group_dequant") is not None:
            raise NotImplementedError("group-wise weight scales take the concatenated input")
        K, N = plan["K"], plan["N"]
        S = self.chunks
        bounds = plan["bounds"]
        xs = []
        for s_, part in enumerate(parts):
            x2 = part.reshape(-1, part.shape[-1])
            if x2.shape[1] != bounds[s_ + 1] - bounds[s_]:
                raise RuntimeError(f"part {s_} has {x2.shape[1]} channels, the segment has {bounds[s_ + 1] - bounds[s_]}")
            xs.append(x2 if x2.is_contiguous() else x2.contiguous())
        M = xs[0].shape[0]
        dev, dt = xs[0].device, xs[0].dtype
        dyn = bool(self.input_calibrators[0].dynamic)
        dual = self.dual_scale
        if dyn:
            pos = torch.empty((S, M), dtype=torch.float32, device=dev)
            neg = torch.empty_like(pos) if dual else None
            per_tok = True
        else:
            pos, neg = self._static_sx(plan, dev)
            per_tok = pos.shape[-1] > 1
            if per_tok and pos.shape[-1] != M:
                raise RuntimeError(f"static per-token scales were calibrated for {pos.shape[-1]} tokens, got {M}")
        fa = plan["fa"]
        codes = torch.empty((M, K), dtype=ops.code_dtype(fa), device=dev)
        codes_neg = torch.empty_like(codes) if dual else None
        ranges = []
        rs = 1 if per_tok else 0
        for s_, x2 in enumerate(xs):
            k0, k1 = bounds[s_], bounds[s_ + 1]
            d_s = bool(dual and self.dual_segments[s_])
            ops.quantize(x2, fa, pos[s_], neg[s_] if d_s else None, row_stride=rs, dual=d_s, dynamic=dyn, two_tensors=d_s,
                         out=codes[:, k0:k1], out_neg=codes_neg[:, k0:k1] if d_s else None, pre_op=pre_ops[s_])
            ranges.append(ops.Range(k0, k1 - k0, pos[s_], plan["sw"], 0, rs, plan["sw_cs"]))
            if d_s:
                ranges.append(ops.Range(k0, k1 - k0, neg[s_], plan["sw"], 1, rs, plan["sw_cs"]))
        g = ops.gemm_desc(codes, plan["w"], ranges, m=M, n=N, a_fmt=fa, b_fmt=plan["fw"], out_dtype=dt, lda=K,
                          ldb=K // 2 if plan["fw"] == ops.FMT_INT4 else K, bias=bias, a_neg=codes_neg)
        int4 = plan["fw"] == ops.FMT_INT4
        ws = None
        if M >= 3072 or not int4:
            need = plan.setdefault("ws_need", {}).get(M)
            if need is None:
                need = plan["ws_need"][M] = ops.gemm_workspace_bytes(g)
            if need:
                ws = ops.int4_workspace(dev, need)
        out = ops.gemm_launch(g, ws)
        return out.view(*parts[0].shape[:-1], N)

    def _relaunch(self, hit, x2, fresh=False):
        """The launches of :meth:`fused_launches` for another input of a token count seen before:
        the cached descriptors with fresh code, scale and output tensors.  (Filling two
        descriptors field by field costs ~30 us of host time per call, which is more than the
        kernels of a small linear take.)"""
        dev = x2.device
        out = torch.empty((hit["M"], hit["N"]), dtype=hit["out_dtype"], device=dev)
        ws = ops.int4_workspace(dev, hit["need"]) if hit["need"] else None
        stream = None
        if not fresh:
            stream = ops._stream(dev)
            bufs = hit.setdefault("buffers", {})
            if stream not in bufs and len(bufs) >= 4 and not torch.cuda.is_current_stream_capturing():
                bufs.pop(next(iter(bufs)))  # streams come and go: keep the buffers of the last few
            reuse = bufs.get(stream)
            if reuse is not None:  # descriptors, codes and scales of the previous call on this stream
                qd, gd, result, held = reuse
                qd.x = x2.data_ptr()
                gd.out = out.data_ptr()
                keep = (x2, out, held)
                return (qd, result, hit["q"][1], keep), (gd, out, hit["g"][1], keep), ws
        # copies of the descriptors: the caller may hold several launches of this layer at once
        qd = type(hit["q"][0]).from_buffer_copy(hit["q"][0])
        gd = type(hit["g"][0]).from_buffer_copy(hit["g"][0])
        codes = torch.empty(hit["code_shape"], dtype=hit["code_dtype"], device=dev)
        qd.x = x2.data_ptr()
        qd.codes = gd.a = codes.data_ptr()
        gd.out = out.data_ptr()
        held = [codes, hit["static"]]
        result = codes
        if hit["dual"]:
            codes_neg = torch.empty_like(codes)
            qd.codes_neg = gd.a_neg = codes_neg.data_ptr()
            held.append(codes_neg)
            result = (codes, codes_neg)
        if hit["dyn"]:
            S, M = hit["S"], hit["M"]
            pos = torch.empty((S, M), dtype=torch.float32, device=dev)
            qd.scale = pos.data_ptr()
            base = [pos.data_ptr(), 0]
            held.append(pos)
            if hit["dual"]:
                neg = torch.empty_like(pos)
                qd.scale_neg = base[1] = neg.data_ptr()
                held.append(neg)
            for i, (which, s_) in enumerate(hit["sx_src"]):
                gd.ranges[i].sx = base[which] + 4 * M * s_
        if stream is not None:
            hit["buffers"][stream] = (qd, gd, result, held)
        keep = (x2, out, held)
        return (qd, result, hit["q"][1], keep), (gd, out, hit["g"][1], keep), ws
