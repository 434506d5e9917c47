"""``quantize(model, calib_loader, config)``: swap ``nn.Linear`` modules for
calibrated ``SegmentLinear`` modules.

Counterpart of segquant/torch/quantization.py:259-425 for the kernel path:
default, smooth and svd optimisers (fixed alpha), amax calibration.  The reference finds segmentation and
DualScale candidates with a torch.fx pattern detector; graph analysis is
outside this build, so both are passed in: ``seg_configs`` maps a linear's name
to ``{"seg_mode", "chunks" | "chunksizes"}`` and ``dual_scale_linears`` names the
linears that follow a SiLU/GELU.
"""
from __future__ import annotations

import fnmatch

import torch
from torch import nn

from ..config import default_quantize_config
from ..layers.SegmentLinear import create_segment_linear


def _move_to_device(batch, device):
    if isinstance(batch, torch.Tensor):
        return batch.to(device)
    if isinstance(batch, (tuple, list)):
        return tuple(_move_to_device(b, device) for b in batch)
    if isinstance(batch, dict):
        return {k: _move_to_device(v, device) for k, v in batch.items()}
    return batch


def _get_all_linears(model: nn.Module, default, config):
    off = [k for k, v in config.items() if k != "default" and v.get("enable") is False]
    on = [k for k, v in config.items() if k != "default" and v.get("enable") is True]
    found = {}
    for name, mod in model.named_modules():
        if not isinstance(mod, nn.Linear):
            continue
        enable = default
        if any(fnmatch.fnmatch(name, p) for p in off):
            enable = False
        if any(fnmatch.fnmatch(name, p) for p in on):
            enable = True
        if enable:
            found[name] = mod
    return found


def _config_for(name, final_config):
    for pattern, cfg in final_config.items():
        if fnmatch.fnmatch(name, pattern):
            return cfg
    return final_config["default"]


def _create_linear(layer: nn.Linear, name, seg, final_config, dual_scale=False, device=None):
    cfg = _config_for(name, final_config)

    def split(key):
        d = dict(cfg[key])
        return d.pop("type"), d

    in_t, in_args = split("input_quant")
    w_t, w_args = split("weight_quant")
    opt_t, opt_args = split("opt")
    cal_t, cal_args = split("calib")
    real = cfg["real_quant"]
    has_bias = layer.bias is not None
    return create_segment_linear(
        in_t, w_t, opt_t, cal_t, layer.in_features, layer.out_features, opt_kwargs=opt_args, calib_kwargs=cal_args,
        input_quant_args={"real_quant": real, "dual_scale": dual_scale, **in_args},
        weight_quant_args={"real_quant": real, **w_args}, bias=has_bias,
        custom_bias_tensor=layer.bias.data if has_bias else None, seg_mode=seg["seg_mode"],
        chunks=seg.get("chunks", len(seg.get("chunksizes", []))), chunksizes=seg.get("chunksizes"),
        custom_weight_tensor=layer.weight.data, device=device)


def _run_model(model, loader, device):
    model.eval()
    with torch.no_grad():
        for batch in loader:
            inp = _move_to_device(batch[0], device)
            model(*inp) if isinstance(inp, tuple) else model(**inp)


def _trace_and_smooth(model, to_smooth, loader, origin_device, target_device):
    """The two extra passes of the smoothing optimisers (reference quantization.py:110-145, :386-412):
    run the calibration data once to record activation maxima, then fix the per-channel factors."""
    hooks = []
    for name, mod in model.named_modules():
        if isinstance(mod, nn.Linear) and name in to_smooth:
            def hook(_m, inp, _out, n=name):
                to_smooth[n].trace(_move_to_device(inp[0], target_device))
            hooks.append(mod.register_forward_hook(hook))
    try:
        _run_model(model, loader, origin_device)
    finally:
        for h in hooks:
            h.remove()
    for lin in to_smooth.values():
        lin.smooth()


def _calib_linears(model, new_linears, loader, origin_device, target_device):
    hooks = []
    for name, mod in model.named_modules():
        if isinstance(mod, nn.Linear) and name in new_linears:
            def hook(_m, inp, _out, n=name):
                new_linears[n].calibrate(_move_to_device(inp[0], target_device))
            hooks.append(mod.register_forward_hook(hook))
    try:
        _run_model(model, loader, origin_device)
    finally:
        for h in hooks:
            h.remove()
    for lin in new_linears.values():
        lin.finish_calibrate()


def _replace_linears(model, new_linears, device):
    for name, lin in new_linears.items():
        parent = model
        *path, leaf = name.split(".")
        for part in path:
            parent = parent[int(part)] if isinstance(parent, (nn.ModuleList, nn.Sequential)) and part.isdigit() \
                else getattr(parent, part)
        if isinstance(parent, (nn.ModuleList, nn.Sequential)) and leaf.isdigit():
            parent[int(leaf)] = lin.to(device)
        else:
            setattr(parent, leaf, lin.to(device))


def quantize(model: nn.Module, calib_data_loader, config=None, tmp_device=None, verbose=False, example=None,
             dump_search=False, search_recovery_file=None, seg_configs=None, dual_scale_linears=None):
    """Quantise ``model`` in place and return it.

    ``calib_data_loader`` yields batches whose first element is the tuple (or
    dict) of model inputs.  ``example``, ``dump_search`` and
    ``search_recovery_file`` are accepted for signature compatibility; they
    belong to the pattern detector and the alpha search, which are not built.
    """
    origin_device = next(model.parameters()).device
    target_device = tmp_device if tmp_device is not None else origin_device
    final_config = dict(config or default_quantize_config)
    final_config.setdefault("default", default_quantize_config["default"])
    if all(not final_config[k]["enable"] for k in final_config):
        return model

    linears = _get_all_linears(model, final_config["default"]["enable"], final_config)
    if verbose:
        print(f"get valid linear num [{len(linears)}]")
    seg_configs = seg_configs or {}
    dual = set(dual_scale_linears or ())
    new_linears = {}
    for name, lin in linears.items():
        seg = {"chunks": 1, "seg_mode": "weight"}
        if name in seg_configs and _config_for(name, final_config).get("seglinear", True):
            seg = seg_configs[name]
        new_linears[name] = _create_linear(lin, name, seg, final_config, dual_scale=name in dual, device=target_device)
    to_smooth = {k: v for k, v in new_linears.items() if v.opt_type in ("smooth", "svd")}
    if to_smooth:
        if verbose:
            print("start trace and smooth ...")
        _trace_and_smooth(model, to_smooth, calib_data_loader, origin_device, target_device)
    if verbose:
        print("start calibrate ...")
    _calib_linears(model, new_linears, calib_data_loader, origin_device, target_device)
    if verbose:
        print("start replace ...")
    _replace_linears(model, new_linears, origin_device)
    if verbose:
        print(model)
    return model
