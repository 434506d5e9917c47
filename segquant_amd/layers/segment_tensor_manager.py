"""Segment views of activations and weights, and the fake-path matmul.

Counterpart of segquant/layers/segment_tensor_manager.py.  The views are what
the reference-convention operators consume; the fused path of this build does
not need them (segments become scale tables and K ranges instead).
"""
import torch


class SegmentTensorManager:
    def __init__(self, seg_mode, segments, segment_size):
        if seg_mode not in ("input", "weight"):
            raise ValueError("seg_mode not found")
        self.seg_mode = seg_mode
        self.segments = segments
        self.segment_size = segment_size


class InputSegmentTensorManager(SegmentTensorManager):
    def __init__(self, input_tensor, seg_mode, segments, segment_size):
        super().__init__(seg_mode, segments, segment_size)
        self.input_tensor = input_tensor

    def iter_view(self):
        """(S, ..., k): input-seg splits the last dim and moves the segment
        index to the front; weight-seg repeats the whole input S times without
        copying (stride 0)."""
        x = self.input_tensor
        if self.seg_mode == "input":
            return x.unflatten(-1, (self.segments, self.segment_size)).movedim(-2, 0)
        return x.unsqueeze(0).expand(self.segments, *x.shape)

    def total_view(self):
        return self.input_tensor.unsqueeze(0)


class WeightSegmentTensorManager(SegmentTensorManager):
    def __init__(self, weight_tensor, seg_mode, segments, segment_size):
        super().__init__(seg_mode, segments, segment_size)
        assert weight_tensor.ndim == 2, "weight tensor shape failed."
        self.out_features, self.in_features = weight_tensor.shape
        self.weight_tensor = weight_tensor
        self.packed = False

    def device(self):
        return self.weight_tensor.device

    def to(self, device):
        self.weight_tensor = self.weight_tensor.to(device)
        return self

    def iter_view(self):
        """(S, n, k) view of the (out, in) weight.  Packed int4 weights are kept
        as (out, in/2) bytes and come back as (S, bytes per segment), the layout
        the reference-convention operators read."""
        w = self.weight_tensor
        if self.packed:
            if self.seg_mode == "input":
                half = self.segment_size // 2
                return w.view(self.out_features, self.segments, half).permute(1, 0, 2).reshape(self.segments, -1)
            return w.view(self.segments, -1)
        if self.seg_mode == "input":
            return w.view(self.out_features, self.segments, self.segment_size).permute(1, 0, 2)
        return w.view(self.segments, self.segment_size, self.in_features)

    def total_view(self):
        return self.weight_tensor.unsqueeze(0)

    def replace_with_segments_layout(self, segmented_weights, packed=False):
        """Store weights given per segment, (S, n, k) or packed (S, bytes), back
        in the (out, in) layout (bytes: (out, in/2))."""
        if packed:
            if self.seg_mode == "input":
                half = self.segment_size // 2
                segmented_weights = segmented_weights.view(self.segments, self.out_features, half).permute(1, 0, 2)
            self.weight_tensor = segmented_weights.reshape(self.out_features, self.in_features // 2).contiguous()
            self.packed = True
            return
        if self.seg_mode == "input":
            segmented_weights = segmented_weights.permute(1, 0, 2).contiguous()
        self.weight_tensor = segmented_weights.reshape(self.out_features, self.in_features)


def segmented_matmul(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """a (S, ..., k) times b (S, n, k) transposed -> (S, ..., n)."""
    assert a.shape[0] == b.shape[0], "segments must match"
    bt = b.transpose(-1, -2)
    while bt.ndim < a.ndim:
        bt = bt.unsqueeze(1)
    return a @ bt
