"""The inference module over the table-batched operators, shaped like the
reference's ``IntNBitTableBatchedEmbeddingBagsCodegen``
(fbgemm_gpu/fbgemm_gpu/split_table_batched_embeddings_ops_inference.py:359-668,
1049-1152, 1705-2010): same constructor arguments, the same weights buffer
(tables concatenated, rows padded to ``row_alignment``, table starts rounded up
to 128 bytes), the same order of work in ``forward`` (bounds check against the
rows before pruning, remap, bounds check against the physical rows, lookup).

Everything lives in one GPU's HBM: the UVM / LXU-cache placements of the
reference are refused. All computation runs in the HIP library.
"""
import enum
from itertools import accumulate

import torch

from . import ops


class SparseType(enum.Enum):
    """fbgemm_gpu/fbgemm_gpu/split_embedding_configs.py; as_int() follows embedding_common.h:20-32."""
    FP32 = "fp32"
    FP16 = "fp16"
    INT8 = "int8"
    INT4 = "int4"
    INT2 = "int2"
    BF16 = "bf16"
    FP8 = "fp8"

    def as_int(self):
        return {"fp32": 0, "fp16": 1, "int8": 2, "int4": 3, "int2": 4, "bf16": 5, "fp8": 6}[self.value]

    def bit_rate(self):
        return {"fp32": 32, "fp16": 16, "int8": 8, "int4": 4, "int2": 2, "bf16": 16, "fp8": 8}[self.value]

    def is_float(self):
        return self.value in ("fp32", "fp16", "bf16", "fp8")


class PoolingMode(enum.IntEnum):
    SUM = 0
    MEAN = 1
    NONE = 2


class BoundsCheckMode(enum.IntEnum):
    FATAL = 0
    WARNING = 1
    IGNORE = 2
    NONE = 3


class EmbeddingLocation(enum.IntEnum):
    DEVICE = 0
    MANAGED = 1
    MANAGED_CACHING = 2
    HOST = 3


def round_up(a, b):
    return (a + b - 1) // b * b


def unpadded_row_size_in_bytes(dim, weight_ty, scale_bias_size_in_bytes=4):
    return ops.unpadded_row_size_in_bytes(dim, weight_ty.as_int(), scale_bias_size_in_bytes)


def rounded_row_size_in_bytes(dim, weight_ty, row_alignment, scale_bias_size_in_bytes=4):
    return ops.padded_row_size_in_bytes(dim, weight_ty.as_int(), row_alignment, scale_bias_size_in_bytes)


class IntNBitTableBatchedEmbeddingBagsCodegen(torch.nn.Module):
    """Table-batched quantized embedding bags for inference on one MI355X."""

    def __init__(self, embedding_specs, feature_table_map=None, index_remapping=None,
                 pooling_mode=PoolingMode.SUM, device=None, bounds_check_mode=BoundsCheckMode.WARNING,
                 weight_lists=None, pruning_hash_load_factor=0.5, use_array_for_index_remapping=True,
                 output_dtype=SparseType.FP16, row_alignment=None, fp8_exponent_bits=None, fp8_exponent_bias=None,
                 scale_bias_size_in_bytes=4,
                 cacheline_alignment=True, reverse_qparam=False, indices_dtype=torch.int32):
        super().__init__()
        self.current_device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        if self.current_device.type != "cuda":
            raise ValueError("this module runs on the GPU; there is no CPU path")
        if scale_bias_size_in_bytes != 4 or reverse_qparam:
            raise NotImplementedError("rows carry an fp16 (scale, bias) pair in front of the elements")
        self.embedding_specs = list(embedding_specs)
        self.pooling_mode = PoolingMode(pooling_mode)
        self.bounds_check_mode_int = int(bounds_check_mode)
        self.output_dtype = output_dtype.as_int()
        self.row_alignment = 16 if row_alignment is None else row_alignment
        self.scale_bias_size_in_bytes = scale_bias_size_in_bytes
        self.indices_dtype = indices_dtype
        self.feature_names = [e[0] for e in self.embedding_specs]
        rows = [e[1] for e in self.embedding_specs]
        dims = [e[2] for e in self.embedding_specs]
        tys = [e[3] for e in self.embedding_specs]
        for e in self.embedding_specs:
            if e[4] not in (EmbeddingLocation.DEVICE, EmbeddingLocation.MANAGED):
                raise NotImplementedError("tables are resident in HBM (DEVICE, or MANAGED = the operator's second weights "
                                          "buffer, kept in HBM too); the UVM cache and host tables are not on this path")
        if self.pooling_mode == PoolingMode.NONE:
            assert all(d == dims[0] for d in dims), "Mixed dimension tables are only supported for pooling tables."
        T_ = len(self.embedding_specs)
        assert T_ > 0
        self.feature_table_map = list(range(T_)) if feature_table_map is None else list(feature_table_map)
        T = len(self.feature_table_map)
        assert T_ <= T
        assert set(self.feature_table_map) == set(range(T_)), "Each table must have at least one feature!"
        for dim, ty in zip(dims, tys):
            if not ty.is_float():
                assert dim % (8 // ty.bit_rate()) == 0, f"quantized rows pack whole bytes: dim {dim}, {ty}"
        D_offsets = [0] + list(accumulate(dims[t] for t in self.feature_table_map))
        self.total_D = D_offsets[-1]

        def max_ty_D(ty):
            return max([d for d, w in zip(dims, tys) if w == ty], default=0)

        self.max_int2_D, self.max_int4_D, self.max_int8_D = max_ty_D(SparseType.INT2), max_ty_D(SparseType.INT4), max_ty_D(SparseType.INT8)
        self.max_float16_D, self.max_float32_D = max(max_ty_D(SparseType.FP16), max_ty_D(SparseType.BF16)), max_ty_D(SparseType.FP32)
        self.max_float8_D = max_ty_D(SparseType.FP8)
        if self.max_float8_D > 0:
            # split_table_batched_embeddings_ops_inference.py: FP8 tables need both parameters
            assert fp8_exponent_bits is not None and fp8_exponent_bias is not None, "FP8 tables need fp8_exponent_bits and fp8_exponent_bias"
        self.fp8_exponent_bits = -1 if fp8_exponent_bits is None else fp8_exponent_bits
        self.fp8_exponent_bias = -1 if fp8_exponent_bias is None else fp8_exponent_bias
        dev = self.current_device
        self.register_buffer("D_offsets", torch.tensor(D_offsets, device=dev, dtype=torch.int32))
        self.register_buffer("rows_per_table", torch.tensor([rows[t] for t in self.feature_table_map], device=dev, dtype=torch.int64))
        self.register_buffer("bounds_check_warning", torch.tensor([0], device=dev, dtype=torch.int64))
        self.register_buffer("weights_tys", torch.tensor([tys[t].as_int() for t in self.feature_table_map], device=dev, dtype=torch.uint8))

        # split_table_batched_embeddings_ops_inference.py:103-147 (nbit_construct_split_state)
        # one running offset per buffer: DEVICE tables in weights_dev, MANAGED ones in weights_uvm
        offsets, sizes, places = [], [0, 0], []
        for _, n, dim, ty, loc in self.embedding_specs:
            state = n * rounded_row_size_in_bytes(dim, ty, self.row_alignment)
            if cacheline_alignment:
                state = round_up(state, 128)
            buf = 1 if loc == EmbeddingLocation.MANAGED else 0
            places.append(buf)
            offsets.append(sizes[buf])
            sizes[buf] += state
        self.dev_size, self.uvm_size = sizes
        self.weights_physical_offsets = offsets
        self.weights_physical_placements = places
        self.register_buffer("weights_offsets", torch.tensor([offsets[t] for t in self.feature_table_map], device=dev, dtype=torch.int64))
        self.register_buffer("weights_placements", torch.tensor([places[t] for t in self.feature_table_map], device=dev, dtype=torch.int32))
        self.weights_dev = torch.zeros(0, device=dev, dtype=torch.uint8)
        self.weights_uvm = torch.zeros(0, device=dev, dtype=torch.uint8)
        self.weight_initialized = False

        self.register_buffer("index_remappings_array_offsets", torch.empty(0, device=dev, dtype=torch.int64))
        self.register_buffer("index_remappings_array", torch.empty(0, device=dev, dtype=indices_dtype))
        self.register_buffer("index_remapping_hash_table_offsets", torch.empty(0, device=dev, dtype=torch.int64))
        self.register_buffer("index_remapping_hash_table", torch.empty(0, device=dev, dtype=indices_dtype))
        self.register_buffer("original_rows_per_table", torch.empty(0, device=dev, dtype=torch.int64))
        if weight_lists:
            self.initialize_weights()
            self.assign_embedding_weights(weight_lists)
        if index_remapping:
            self.set_index_remappings(index_remapping, pruning_hash_load_factor, use_array_for_index_remapping)

    # ---- weights -------------------------------------------------------------
    def initialize_weights(self):
        if not self.weight_initialized:
            self.weights_dev = torch.zeros(self.dev_size, device=self.current_device, dtype=torch.uint8)
            self.weights_uvm = torch.zeros(self.uvm_size, device=self.current_device, dtype=torch.uint8)
            self.weight_initialized = True

    def split_embedding_weights_with_scale_bias(self, split_scale_bias_mode=1):
        """Per table: 0: (whole padded rows, None, None); 1: (elements, fp16 pair as bytes, None);
        2: (elements, scale, bias). Views into the weights buffer."""
        assert self.weight_initialized
        splits = []
        for t, (_, n, dim, ty, _) in enumerate(self.embedding_specs):
            rb = rounded_row_size_in_bytes(dim, ty, self.row_alignment)
            off = self.weights_physical_offsets[t]
            buf = self.weights_uvm if self.weights_physical_placements[t] else self.weights_dev
            w = buf.detach()[off:off + n * rb].view(n, rb)
            if split_scale_bias_mode == 0:
                splits.append((w, None, None))
                continue
            w = w[:, :unpadded_row_size_in_bytes(dim, ty)]
            if ty.is_float():
                splits.append((w, None, None))
            elif split_scale_bias_mode == 1:
                splits.append((w[:, 4:], w[:, :4], None))
            elif split_scale_bias_mode == 2:
                splits.append((w[:, 4:], w[:, :2].view(torch.float16), w[:, 2:4].view(torch.float16)))
            else:
                raise ValueError("split_scale_bias_mode is not supported")
        return splits

    def split_embedding_weights(self, split_scale_shifts=True):
        return [(s[0], s[1]) for s in self.split_embedding_weights_with_scale_bias(1 if split_scale_shifts else 0)]

    def fill_random_weights(self):
        """Random bytes in the element part of every row, as the reference fills them
        (random_quant_scaled_tensor: bytes in [0, 255))."""
        self.initialize_weights()
        for dest, _ in self.split_embedding_weights():
            dest.copy_(torch.randint(0, 255, size=dest.shape, dtype=torch.uint8, device=self.current_device))

    def assign_embedding_weights(self, q_weight_list):
        weights = self.split_embedding_weights()
        assert len(q_weight_list) == len(weights)
        for dest, src in zip(weights, q_weight_list):
            dest[0].copy_(src[0])
            if src[1] is not None:
                assert dest[1] is not None
                dest[1].copy_(src[1].view(torch.uint8) if src[1].dtype != torch.uint8 else src[1])
            else:
                assert dest[1] is None

    def quantize_and_assign(self, fp_weight_list, fp8_max_position=None):
        """fp32 / fp16 tables -> this module's rows, on the GPU (the producer the
        reference runs on the CPU: tbe/utils/quantize.py:20-72). FP8 tables take the
        clamp of FP8QuantizationConfig (``fp8_max_position``; default: the largest
        value the format holds below its top exponent)."""
        self.initialize_weights()
        assert len(fp_weight_list) == len(self.embedding_specs)
        rows = self.split_embedding_weights_with_scale_bias(0)
        for (whole, _, _), src, (_, n, dim, ty, _) in zip(rows, fp_weight_list, self.embedding_specs):
            src = src.to(self.current_device)
            assert tuple(src.shape) == (n, dim)
            if ty.is_float():
                if ty == SparseType.FP8:
                    eb, bias = self.fp8_exponent_bits, self.fp8_exponent_bias
                    max_pos = fp8_max_position
                    if max_pos is None:  # split_embedding_configs.py:317-318
                        max_pos = (1 << ((1 << eb) - 2 - bias)) * (2 - 2 ** (eb - 7))
                    whole[:, :dim].copy_(ops.float_to_hfp8_quantized(src.float(), eb, bias, max_pos))
                    continue
                want = {SparseType.FP32: torch.float32, SparseType.FP16: torch.float16, SparseType.BF16: torch.bfloat16}[ty]
                whole[:, :dim * ty.bit_rate() // 8].copy_(src.to(want).contiguous().view(torch.uint8).view(n, -1))
            else:
                ops.quantize_rowwise(src if src.dtype == torch.float16 else src.float(), ty.bit_rate(), False,
                                     ops.QLAYOUT_TBE, out=whole)

    # ---- pruning ---------------------------------------------------------------
    def set_index_remappings_array(self, index_remapping):
        rows = [e[1] for e in self.embedding_specs]
        offs, original, last = [0], [], 0
        for t, mapping in enumerate(index_remapping):
            if mapping is not None:
                last += mapping.numel()
                original.append(mapping.numel())
            else:
                original.append(rows[t])
            offs.append(last)
        dev = self.current_device
        self.index_remappings_array_offsets = torch.tensor(offs, device=dev, dtype=torch.int64)
        self.original_rows_per_table = torch.tensor([original[t] for t in self.feature_table_map], device=dev, dtype=torch.int64)
        kept = [m for m in index_remapping if m is not None]
        self.index_remappings_array = (torch.cat(kept).to(dtype=self.indices_dtype, device=dev) if kept
                                       else torch.empty(0, dtype=self.indices_dtype, device=dev))
        # The lookups address a mapping slice per FEATURE (offsets[f], offsets[f + 1]), the arrays above hold
        # one per TABLE, as the reference's do (its own pruned_array_lookup derives the batch size from them and
        # so does not support features that share a pruned table). With shared tables the forward gets a
        # per-feature copy of the slices; without, the very same tensors.
        ftm = list(self.feature_table_map)
        if ftm == list(range(len(self.embedding_specs))) or not kept:
            self._feature_remap_array = self.index_remappings_array
            self._feature_remap_offsets = (self.index_remappings_array_offsets if kept else
                                           torch.zeros(len(ftm) + 1, device=dev, dtype=torch.int64))
        else:
            parts, foffs = [], [0]
            for t in ftm:
                if index_remapping[t] is not None:
                    parts.append(index_remapping[t].to(dtype=self.indices_dtype, device=dev))
                foffs.append(foffs[-1] + (index_remapping[t].numel() if index_remapping[t] is not None else 0))
            self._feature_remap_array = torch.cat(parts)
            self._feature_remap_offsets = torch.tensor(foffs, device=dev, dtype=torch.int64)

    def set_index_remappings(self, index_remapping, pruning_hash_load_factor=0.5, use_array_for_index_remapping=True):
        if use_array_for_index_remapping:
            return self.set_index_remappings_array(index_remapping)
        rows = [e[1] for e in self.embedding_specs]
        capacities = [round_up(int(r / pruning_hash_load_factor), 32) if m is not None else 0
                      for m, r in zip(index_remapping, rows)]
        hash_table = torch.full((sum(capacities), 2), -1, dtype=self.indices_dtype)
        hto = torch.tensor([0] + list(accumulate(capacities)), dtype=torch.int64)
        merged = [m.cpu() if m is not None else torch.arange(r) for m, r in zip(index_remapping, rows)]
        original = [m.numel() for m in merged]
        dev = self.current_device
        self.original_rows_per_table = torch.tensor([original[t] for t in self.feature_table_map], device=dev, dtype=torch.int64)
        dense = torch.cat(merged).to(self.indices_dtype)
        indices = torch.cat([torch.arange(r) for r in original]).to(self.indices_dtype)
        offsets = torch.tensor([0] + list(accumulate(original))).to(self.indices_dtype)
        ops.pruned_hashmap_insert(indices, dense, offsets, hash_table, hto)
        self.index_remapping_hash_table = hash_table.to(dev)
        self.index_remapping_hash_table_offsets = hto.to(dev)

    # ---- in-place updates ------------------------------------------------------
    def _embedding_inplace_update_per_table(self, update_table_idx, update_row_indices, update_weights):
        # split_table_batched_embeddings_ops_inference.py:2018-2041: whole padded rows, scattered by row id
        if len(update_row_indices) == 0:
            return
        rows = torch.tensor(update_row_indices, device=self.current_device, dtype=torch.int64)
        table = self.split_embedding_weights(split_scale_shifts=False)[update_table_idx][0]
        table.scatter_(dim=0, index=rows.view(-1, 1).expand_as(update_weights), src=update_weights)

    def embedding_inplace_update(self, update_table_indices, update_row_indices, update_weights):
        """Per table: a list of rows and a [rows, padded row bytes] uint8 tensor
        (split_table_batched_embeddings_ops_inference.py:2044-2055)."""
        for t, rows, w in zip(update_table_indices, update_row_indices, update_weights):
            self._embedding_inplace_update_per_table(t, rows, w)

    def embedding_inplace_update_internal(self, update_table_indices, update_row_indices, update_weights):
        """Flat form: update i overwrites row update_row_indices[i] (a logical row when the module prunes
        through arrays) of table update_table_indices[i] with the next padded row of ``update_weights``
        (split_table_batched_embeddings_ops_inference.py:2057-2144). One kernel for all tables."""
        assert len(update_table_indices) == len(update_row_indices)
        dev = self.current_device
        sizes = [rounded_row_size_in_bytes(self.embedding_specs[t][2], self.embedding_specs[t][3], self.row_alignment,
                                           self.scale_bias_size_in_bytes) for t in update_table_indices]
        update_offsets = torch.tensor([0] + list(accumulate(sizes)), device=dev, dtype=torch.int64)
        tables = torch.tensor(update_table_indices, device=dev, dtype=torch.int32)
        rows = torch.tensor(update_row_indices, device=dev, dtype=torch.int64)
        # only array based pruning, as in the reference
        assert self.index_remapping_hash_table.numel() == 0
        if self.index_remappings_array.numel() > 0:
            rows = ops.pruned_array_lookup_from_row_idx(rows, tables, self.index_remappings_array,
                                                        self.index_remappings_array_offsets)
        # the operator addresses weights_offsets, which has one entry per feature: the first feature of each table
        first_feature = [self.feature_table_map.index(t) for t in range(len(self.embedding_specs))]
        features = torch.tensor([first_feature[t] for t in update_table_indices], device=dev, dtype=torch.int32)
        ops.emb_inplace_update(self.weights_dev, self.weights_uvm, self.weights_placements, self.weights_offsets,
                               self.weights_tys, self.D_offsets, update_weights.to(dev), features, rows, update_offsets,
                               row_alignment=self.row_alignment)

    # ---- forward ---------------------------------------------------------------
    def forward(self, indices, offsets, per_sample_weights=None):
        assert self.weight_initialized, "weight needs to be initialized before forward function"
        dev = self.current_device
        indices, offsets = indices.to(dev), offsets.to(dev)
        if per_sample_weights is not None:
            per_sample_weights = per_sample_weights.to(dev)
        check = self.bounds_check_mode_int != BoundsCheckMode.NONE.value
        hashed = self.index_remapping_hash_table.numel() > 0
        arrayed = self.index_remappings_array.numel() > 0
        fuse_remap = arrayed and not check and self.pooling_mode != PoolingMode.NONE
        if check and (hashed or arrayed or self.bounds_check_mode_int != BoundsCheckMode.FATAL.value):
            # in-place repairs must not reach the caller's tensors
            indices, offsets = indices.clone(), offsets.clone()
        if (hashed or arrayed) and check:
            ops.bounds_check_indices(self.original_rows_per_table, indices, offsets, self.bounds_check_mode_int,
                                     self.bounds_check_warning, per_sample_weights)
        if hashed:
            indices = ops.pruned_hashmap_lookup(indices, offsets, self.index_remapping_hash_table,
                                                self.index_remapping_hash_table_offsets)
        elif arrayed and not fuse_remap:
            indices = ops.pruned_array_lookup(indices, offsets, self._feature_remap_array, self._feature_remap_offsets)
        if check:
            ops.bounds_check_indices(self.rows_per_table, indices, offsets, self.bounds_check_mode_int,
                                     self.bounds_check_warning, per_sample_weights)
        return ops.int_nbit_split_embedding_codegen_lookup_function(
            self.weights_dev, self.weights_uvm, self.weights_placements, self.weights_offsets, self.weights_tys,
            self.D_offsets, self.total_D, self.max_int2_D, self.max_int4_D, self.max_int8_D, self.max_float16_D,
            self.max_float32_D, indices, offsets, int(self.pooling_mode), per_sample_weights, self.output_dtype,
            row_alignment=self.row_alignment, max_float8_D=self.max_float8_D,
            fp8_exponent_bits=self.fp8_exponent_bits, fp8_exponent_bias=self.fp8_exponent_bias,
            index_remappings=self._feature_remap_array if fuse_remap else None,
            index_remappings_offsets=self._feature_remap_offsets if fuse_remap else None)
