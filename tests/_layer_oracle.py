"""Closed form of a calibrated SegmentLinear's fused forward, built with the CPU
oracle from the layer's stored weight codes and scales (test helper)."""
import numpy as np
import torch

from oracle import segq_oracle as O


def _np32(t):
    return t.detach().float().cpu().numpy()


def _unpacked_weight_codes(layer, fmt):
    w = layer.optimizer.weight_manager.weight_tensor.cpu().numpy()
    if fmt == O.FMT_INT4:
        return np.stack([O.unpack_int4(r) for r in w])
    return w


def _scale_fn(fmt):
    bits = 4 if fmt == O.FMT_INT4 else 8
    if fmt == O.FMT_E4M3:
        return O.fp8_scale, O.fp8_dual_scales
    return (lambda a: O.int_scale(a, bits)), (lambda p, n: O.int_dual_scales(p, n, bits))


def oracle_layer_output(layer, spec, x_np, out_dtype=None, rows=None, cols=None):
    """Closed form of the fused forward from the layer's stored codes and scales, in fp64.

    ``rows`` / ``cols``: index lists restricting the result to a band of tokens or of output
    columns (full-size shapes are checked on bands: the oracle cannot multiply them whole in
    seconds).  Static per-token activation scales are not banded (no configuration uses them)."""
    from segquant_amd.workloads import segment_bounds
    opt = layer.optimizer
    fa, fw = spec.act, spec.weight
    wq = _unpacked_weight_codes(layer, fw)
    if rows is not None:
        x_np = x_np[np.asarray(rows)]
    N_all = wq.shape[0]
    csel = np.arange(N_all) if cols is None else np.asarray(cols)
    wq = wq[csel]
    N, K = wq.shape
    M = x_np.shape[0]
    bounds = segment_bounds(spec)
    single, dualf = _scale_fn(fa)
    # weight scale per output column, or per (column, group of input channels)
    wcals = opt.weight_calibrators
    group = getattr(wcals[0], "group_size", None)
    if group:
        sw_groups = np.concatenate([_np32(c.scale).reshape(-1, K // group) for c in wcals]).astype(np.float32)[csel]
        sw = None
    elif spec.seg_mode == "weight" and len(wcals) > 1:
        sw = np.concatenate([np.broadcast_to(np.float32(_np32(torch.as_tensor(c.scale))).reshape(-1), (n,)) if
                             np.ndim(c.scale) == 0 or torch.as_tensor(c.scale).numel() == 1 else
                             _np32(c.scale) for c, n in zip(wcals, opt.chunksizes)])
    else:
        s0 = torch.as_tensor(wcals[0].scale).float().cpu().numpy().reshape(-1)
        sw = np.broadcast_to(s0, (N_all,)) if s0.size == 1 else s0
    if sw is not None:
        sw = sw.astype(np.float32)[csel].reshape(1, N)

    def dequantised(codes, k0, k1, sx):
        """sum over the weight-scale blocks of [k0, k1) of acc / (sx * sw)"""
        if not group:
            return O.gemm_acc(codes, wq[:, k0:k1], fa, fw) / (sx.astype(np.float64) * sw)
        t = np.zeros((M, N), dtype=np.float64)
        for g0 in range(k0, k1, group):
            swg = sw_groups[:, g0 // group].reshape(1, N)
            t += O.gemm_acc(codes[:, g0 - k0:g0 - k0 + group], wq[:, g0:g0 + group], fa, fw) / (sx.astype(np.float64) * swg)
        return t

    y = np.zeros((M, N), dtype=np.float64)
    for s in range(len(bounds) - 1):
        k0, k1 = bounds[s], bounds[s + 1]
        xs = x_np[:, k0:k1]
        cal = opt.input_calibrators[s if spec.seg_mode == "input" else 0]
        dual = opt.dual_segments[s if spec.seg_mode == "input" else 0]
        if spec.dynamic:  # the kernel's own definition: one fp32 division per row
            lim_p = {O.FMT_INT8: 127.0, O.FMT_INT4: 7.0, O.FMT_E4M3: 448.0}[fa]
            lim_n = {O.FMT_INT8: 128.0, O.FMT_INT4: 8.0, O.FMT_E4M3: 448.0}[fa]
            if dual:
                pa, na = O.dual_amax(xs, axis=-1)
                ps, ns = O.row_scale_div(pa, lim_p), O.row_scale_div(na, lim_n)
            else:
                ps = O.row_scale_div(np.abs(xs).max(axis=-1), lim_p)
        else:
            if dual:
                ps, ns = (np.float32(_np32(torch.as_tensor(t))) for t in (cal.pos_scale, cal.neg_scale))
            else:
                ps = np.float32(_np32(torch.as_tensor(cal.scale)))
        ps = np.float32(ps).reshape(-1)
        psb = ps.reshape(-1, 1) if ps.size > 1 else ps.reshape(1, 1)
        if dual:
            ns = np.float32(ns).reshape(-1)
            nsb = ns.reshape(-1, 1) if ns.size > 1 else ns.reshape(1, 1)
            cp, cn = O.quantize_act_dual(xs[None], ps if ps.size > 1 else ps[:1], ns if ns.size > 1 else ns[:1], fa)
            y += dequantised(cp[0], k0, k1, psb)
            y += dequantised(cn[0], k0, k1, nsb)
        else:
            c = O.quantize_act(xs[None], ps if ps.size > 1 else ps[:1], fa)
            y += dequantised(c[0], k0, k1, psb)
    if layer.bias:
        y += _np32(layer.bias_data).astype(np.float64)[csel]
    return y


def oracle_smooth_layer_output(layer, fmt_a, fmt_w, x_np, rows=None, cols=None):
    """Closed form (fp64) of a calibrated smooth / svd SegmentLinear with input segmentation or a
    single chunk, from the layer's own factors, codes and scales: per K segment i,
    codes(x_i / s_i) W_i^T / (sx_i sw_i) + (x_i / s_i) L1_i L2_i, plus the bias
    (segquant/optimum/optimizer.py:514-517, :724-731).  The division is carried out in the
    input's dtype grid when ``x_np`` holds bf16 / fp16 values (``dtype`` of the layer's input)."""
    opt = layer.optimizer
    wq = _unpacked_weight_codes(layer, fmt_w)
    if rows is not None:
        x_np = x_np[np.asarray(rows)]
    csel = np.arange(wq.shape[0]) if cols is None else np.asarray(cols)
    wq = wq[csel]
    N, K = wq.shape
    S = opt.chunks if opt.seg_mode == "input" else 1
    ksz = K // S
    y = np.zeros((x_np.shape[0], N))
    lim = {O.FMT_INT8: 127.0, O.FMT_E4M3: 448.0}[fmt_a]
    for i in range(S):
        ks = slice(i * ksz, (i + 1) * ksz)
        s = _np32(opt.s[i]).astype(np.float32)
        xs = O.smooth_divide(x_np[:, ks], s, layer._oracle_dtype)
        cal = opt.input_calibrators[i]
        if cal.dynamic:
            sx = O.row_scale_div(np.abs(xs).max(axis=-1), lim)
        else:
            sx = np.float32(_np32(torch.as_tensor(cal.scale))).reshape(-1)
        sw = np.float32(_np32(torch.as_tensor(opt.weight_calibrators[i].scale))).reshape(-1)
        sw = (np.broadcast_to(sw, (layer.out_features,)) if sw.size == 1 else sw)[csel].astype(np.float64)
        codes = O.quantize_act(xs[None], sx if sx.size > 1 else sx[:1], fmt_a)[0]
        y += O.gemm_acc(codes, wq[:, ks], fmt_a, fmt_w) / (sx.astype(np.float64).reshape(-1, 1) * sw[None, :])
        if getattr(opt, "l1s", None) is not None:
            l1 = _np32(opt.l1s[i]).astype(np.float64)
            l2 = _np32(opt.l2s[i]).astype(np.float64)[:, csel]
            y += (xs.astype(np.float64) @ l1) @ l2
    if layer.bias:
        y += _np32(layer.bias_data).astype(np.float64)[csel]
    return y
