"""Gradient compression as seen by the callers of allreduce.

Same interface as horovod/torch/compression.py:20-74: a compressor turns a tensor into the
tensor that travels plus a context, and back.  Used on their own the classes behave like the
reference's (fp16 = a framework cast each way).  The allreduce entry points of this package
recognise ``Compression.fp16`` on float32 device tensors and skip both casts and both
temporaries: the narrowing is done by the kernel that packs the fusion buffer and the widening
by the one that unpacks it, with the roundings of the two-step pipeline.
"""
import torch


class Compressor(object):
    """compress(tensor) -> (tensor_on_the_wire, ctx); decompress(tensor, ctx) -> tensor."""

    @staticmethod
    def compress(tensor):
        raise NotImplementedError

    @staticmethod
    def decompress(tensor, ctx):
        raise NotImplementedError


class NoneCompressor(Compressor):
    @staticmethod
    def compress(tensor):
        return tensor, None

    @staticmethod
    def decompress(tensor, ctx):
        return tensor


class FP16Compressor(Compressor):
    """Floating-point tensors travel as float16; everything else is left alone."""

    @staticmethod
    def compress(tensor):
        # the context is the dtype to come back to
        travels = tensor.to(torch.float16) if tensor.dtype.is_floating_point else tensor
        return travels, tensor.dtype

    @staticmethod
    def decompress(tensor, ctx):
        return tensor.to(ctx) if ctx.is_floating_point else tensor

    @staticmethod
    def fuses_into_packing(tensor):
        """True where the cast can ride on the pack/unpack kernels (float32 on the GPU)."""
        return tensor.is_cuda and tensor.dtype == torch.float32


class Compression(object):
    none = NoneCompressor
    fp16 = FP16Compressor
