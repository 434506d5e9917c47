"""MI355X-native real-quantised segmented linear (the SegQuant hot path).

``segquant_amd.ops`` wraps the C ABI of ``libsegq.so`` (hand-written HIP for
gfx950); ``segquant_amd.layers`` mirrors the reference's segmented-linear
module and its ``ext_dict`` registry on top of it.
"""
__version__ = "0.1.0"
