"""The inference converter: float tables -> pruned, quantized rows inside an
``IntNBitTableBatchedEmbeddingBagsCodegen``, all on the GPU.

Mirrors ``SplitEmbInferenceConverter``
(fbgemm_gpu/fbgemm_gpu/split_embedding_inference_converter.py:37-164) and
``quantize_embs`` (fbgemm_gpu/fbgemm_gpu/tbe/utils/quantize.py:20-72): rows are
ranked by their L2 norm, the smallest ``pruning_ratio`` of them are dropped with
``embedding_bag_rowwise_prune`` (which leaves the remap array the lookups need),
the rest are quantized row by row. The reference moves every table to the host
for this; here the tables stay in HBM. The row norms are fp32 sums computed by
torch on the device, so they can differ from numpy's in the last place; the
prune and the quantizers themselves reproduce the reference's results bit for bit.
"""
import math

import torch

from . import ops
from .module import EmbeddingLocation, IntNBitTableBatchedEmbeddingBagsCodegen, PoolingMode, SparseType

ALIGN_SIZE = {SparseType.FP32: 1, SparseType.FP16: 2, SparseType.BF16: 2, SparseType.FP8: 4, SparseType.INT8: 4,
              SparseType.INT4: 8, SparseType.INT2: 16}  # split_embedding_configs.py:471-482


class QuantizationConfig:
    def get(self, name):
        return -1


class FP8QuantizationConfig(QuantizationConfig):
    """split_embedding_configs.py:311-324."""

    def __init__(self, exponent_bits, exponent_bias):
        self.config = {"exponent_bits": exponent_bits, "exponent_bias": exponent_bias,
                       "max_position": (1 << ((1 << exponent_bits) - 2 - exponent_bias)) * (2 - 2 ** (exponent_bits - 7))}

    def get(self, name):
        if name not in self.config:
            raise RuntimeError(f"{name} must be set in config")
        return self.config[name]


def quantize_embs(weight, weight_ty, fp8_config=None):
    """quantize_embs (tbe/utils/quantize.py:20-72): (row bytes, fp16 scale/bias bytes or None)."""
    weight = weight.detach()
    if weight_ty == SparseType.FP32:
        return weight.float().contiguous().view(torch.uint8), None
    if weight_ty == SparseType.FP16:
        return weight.half().contiguous().view(torch.uint8), None
    if weight_ty == SparseType.FP8:
        assert fp8_config is not None
        return ops.float_to_hfp8_quantized(weight.float(), fp8_config.get("exponent_bits"), fp8_config.get("exponent_bias"),
                                           fp8_config.get("max_position")), None
    if weight_ty == SparseType.INT8:
        q = ops.quantize_rowwise(weight.float(), 8, True)
        sb = q[:, -8:].contiguous().view(torch.float32).to(torch.float16).view(torch.uint8)
        return q[:, :-8], sb
    if weight_ty in (SparseType.INT4, SparseType.INT2):
        q = ops.quantize_rowwise(weight.float(), weight_ty.bit_rate(), False)
        return q[:, :-4], q[:, -4:]
    raise RuntimeError(f"Unsupported SparseType: {weight_ty}")


class SplitEmbInferenceConverter:
    def __init__(self, quantize_type, pruning_ratio, use_array_for_index_remapping=True, quantization_config=None):
        self.quantize_type = quantize_type
        self.pruning_ratio = pruning_ratio
        self.use_array_for_index_remapping = use_array_for_index_remapping
        self.quantization_config = quantization_config

    def _prune_by_weights_l2_norm(self, new_num_rows, weights):
        """(row norms, threshold): the largest norm strictly below the norm of the last row to keep."""
        assert new_num_rows > 0
        indicators = torch.linalg.vector_norm(weights.float(), ord=2, dim=1)
        ordered = torch.sort(indicators, descending=True).values
        below = ordered[new_num_rows:][ordered[new_num_rows:] < ordered[new_num_rows - 1]]
        threshold = float(below[0]) if below.numel() else float(ordered[-1]) - 1
        return indicators, threshold

    def _prune_embs(self, weights):
        num_rows = weights.size(0)
        if self.pruning_ratio is None:
            return weights, None
        new_num_rows = int(math.ceil(num_rows * (1.0 - self.pruning_ratio)))
        if new_num_rows == num_rows:
            return weights, None
        indicators, threshold = self._prune_by_weights_l2_norm(new_num_rows, weights)
        return ops.embedding_bag_rowwise_prune(weights, indicators, threshold, torch.int32)

    def _quantize_embs(self, weight, weight_ty):
        return quantize_embs(weight, weight_ty, self.quantization_config)

    def convert_tables(self, weights, pooling_mode=PoolingMode.SUM, **module_args):
        """Float tables ``[E_t, D_t]`` on the GPU -> the inference module holding them pruned and quantized."""
        specs, weight_lists, remaps = [], [], []
        for w in weights:
            if not w.is_cuda:
                raise ValueError("the converter works on device tensors; there is no CPU path")
            D = w.size(1)
            ty = self.quantize_type
            if D % ALIGN_SIZE[ty] != 0:
                assert D % 4 == 0
                ty = SparseType.FP16  # the reference's fall-back when the dimension does not fit the type
            pruned, remap = self._prune_embs(w)
            specs.append(("", pruned.size(0), D, ty, EmbeddingLocation.DEVICE))
            remaps.append(remap)
            weight_lists.append(quantize_embs(pruned, ty, self.quantization_config))
        is_fp8 = self.quantize_type == SparseType.FP8
        if is_fp8 and self.quantization_config is None:
            raise RuntimeError("quantization_config must be set for FP8 weight")
        return IntNBitTableBatchedEmbeddingBagsCodegen(
            embedding_specs=specs, index_remapping=remaps if self.pruning_ratio is not None else None,
            pooling_mode=pooling_mode, device=weights[0].device, weight_lists=weight_lists,
            use_array_for_index_remapping=self.use_array_for_index_remapping,
            fp8_exponent_bits=self.quantization_config.get("exponent_bits") if is_fp8 else None,
            fp8_exponent_bias=self.quantization_config.get("exponent_bias") if is_fp8 else None, **module_args)

    def convert_model(self, model):
        """Replace every child that holds float tables the way the reference's training module does
        (``split_embedding_weights()`` returning the tables, ``pooling_mode``) with the converted module."""
        for name, child in model.named_children():
            if hasattr(child, "split_embedding_weights") and not isinstance(child, IntNBitTableBatchedEmbeddingBagsCodegen):
                tables = [w.to("cuda") for w in child.split_embedding_weights()]
                setattr(model, name, self.convert_tables(tables, PoolingMode(int(child.pooling_mode))))
            else:
                self.convert_model(child)
        return model
