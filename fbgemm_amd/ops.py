"""Python face of the C ABI, shaped like the reference's own entry points.

* ``generate_embedding_spmdm*`` mirror the kernel factories of
  include/fbgemm/FbgemmEmbedding.h:65-262: fix the configuration once, get back
  a callable with the ``EmbeddingSpMDMKernelSignature`` argument list that
  returns the reference's ``bool``.
* ``int_nbit_split_embedding_codegen_lookup_function`` and
  ``pruned_array_lookup`` mirror the operators registered in
  fbgemm_gpu/codegen/inference/embedding_forward_quantized_host_cpu.cpp:310-347.

All tensors are device tensors (torch is only the owner of HBM and streams).
Everything runs in the HIP library; nothing here computes.
"""
import collections
import ctypes as C

import torch

from . import _lib
from ._lib import SpmdmConfig, check

FP32, FP16, INT8, INT4, INT2, BF16, FP8 = 0, 1, 2, 3, 4, 5, 6
POOL_SUM, POOL_MEAN, POOL_NONE = 0, 1, 2
ACC_EXACT, ACC_FAST = 0, 1  # how 4- and 8-bit rows are accumulated (include/fbgemm_amd.h)

_OUT_TORCH = {FP32: torch.float32, FP16: torch.float16, BF16: torch.bfloat16}
_TORCH_OUT = {v: k for k, v in _OUT_TORCH.items()}

ERR_INDEX_OUT_OF_RANGE, ERR_BAG_OVERRUN, ERR_LENGTH_MISMATCH, ERR_NEGATIVE_LENGTH = 1, 2, 4, 8


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _bits(t):
    if t.dtype == torch.int64:
        return 64
    if t.dtype == torch.int32:
        return 32
    raise TypeError(f"indices/offsets must be int32 or int64, got {t.dtype}")


def _require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("fbgemm_amd ops take device tensors; there is no CPU path")


class Status:
    """A device status block (see include/fbgemm_amd.h)."""

    def __init__(self, device=None):
        self.buf = torch.zeros(4, dtype=torch.int32, device=device or "cuda")
        self.clear()

    def clear(self):
        check(_lib.lib().fbgemm_amd_status_clear(_ptr(self.buf), _stream()))

    def read(self):
        """Synchronizes. Returns (bits, first_bad_pos)."""
        bits, pos = C.c_int32(0), C.c_int64(-1)
        check(_lib.lib().fbgemm_amd_status_read(_ptr(self.buf), _stream(), C.byref(bits), C.byref(pos)))
        return bits.value, pos.value


def _make_kernel(weight_ty, block_size, normalize_by_lengths, is_weight_positional, use_offsets,
                 output_stride, input_stride, scale_bias_last, output_ty, has_weight, sparse, no_bag=False,
                 fp8=(0, 0)):
    def kernel(output_size, index_size, data_size, input, indices, offsets_or_lengths, weights, out,
               compressed_indices_table=None, status=None, accumulate=ACC_EXACT):
        _require_cuda(input, indices, offsets_or_lengths, weights, out, compressed_indices_table)
        if sparse and compressed_indices_table is None:
            raise ValueError("row-wise-sparse kernels need compressed_indices_table")
        if has_weight is not None and has_weight != (weights is not None):
            # the reference's generated code is specialised on has_weight; a mismatch is a caller bug
            raise ValueError("weights must be given exactly when has_weight was set")
        if weights is not None and weights.dtype != torch.float32:
            raise TypeError("weights must be float32")
        if compressed_indices_table is not None and compressed_indices_table.dtype != torch.int32:
            raise TypeError("compressed_indices_table must be int32")
        cfg = SpmdmConfig(
            weight_ty=weight_ty, output_ty=output_ty, index_bits=_bits(indices),
            offset_bits=32 if offsets_or_lengths is None else _bits(offsets_or_lengths), block_size=block_size,
            output_stride=output_stride, input_stride=input_stride,
            normalize_by_lengths=int(normalize_by_lengths),
            is_weight_positional=int(is_weight_positional), use_offsets=int(use_offsets),
            scale_bias_last=int(scale_bias_last), no_bag=int(no_bag), fp8_exponent_bits=fp8[0],
            fp8_exponent_bias=fp8[1], accumulate=int(accumulate))
        lib = _lib.lib()
        if status is not None:
            check(lib.fbgemm_amd_spmdm_launch(
                C.byref(cfg), output_size, index_size, data_size, _ptr(input), _ptr(indices),
                _ptr(offsets_or_lengths), _ptr(weights), _ptr(out), _ptr(compressed_indices_table),
                _ptr(status.buf), _stream()))
            return None
        rc = check(lib.fbgemm_amd_spmdm_run(
            C.byref(cfg), output_size, index_size, data_size, _ptr(input), _ptr(indices),
            _ptr(offsets_or_lengths), _ptr(weights), _ptr(out), _ptr(compressed_indices_table),
            _stream()))
        return rc == 1

    return kernel


def generate_embedding_spmdm_with_strides(
        in_ty, block_size, has_weight, normalize_by_lengths, prefetch=16,
        is_weight_positional=False, use_offsets=True, output_stride=-1, input_stride=-1,
        scale_bias_last=True, no_bag=False, is_bf16_out=False, is_bf16_in=False, out_ty=FP32):
    """GenerateEmbeddingSpMDMWithStrides (FbgemmEmbedding.h:94-117). ``in_ty`` is
    INT8 (fused 8-bit rows), FP16 or FP32; ``out_ty`` FP32 or FP16 (BF16 via
    ``is_bf16_out``). ``prefetch`` is accepted and ignored: the GPU hides
    latency with loads in flight, not software prefetch. With ``no_bag`` the
    kernel writes one row per index (``offsets_or_lengths`` may be None) and
    ``out_ty`` INT8 copies the rows as stored (the reference's uint8_t output)."""
    if in_ty == FP16 and is_bf16_in:
        in_ty = BF16
    if is_bf16_out:
        out_ty = BF16
    return _make_kernel(in_ty, block_size, normalize_by_lengths, is_weight_positional, use_offsets,
                        output_stride, input_stride, scale_bias_last, out_ty, has_weight, False, no_bag)


def generate_embedding_spmdm(in_ty, block_size, has_weight, normalize_by_lengths, prefetch=16,
                             is_weight_positional=False, use_offsets=True, is_bf16_out=False,
                             is_bf16_in=False, out_ty=FP32):
    """GenerateEmbeddingSpMDM (FbgemmEmbedding.h:65-84)."""
    return generate_embedding_spmdm_with_strides(
        in_ty, block_size, has_weight, normalize_by_lengths, prefetch, is_weight_positional,
        use_offsets, -1, -1, True, False, is_bf16_out, is_bf16_in, out_ty)


def generate_embedding_spmdm_nbit_with_strides(
        input_bit_rate, block_size, has_weight, normalize_by_lengths, prefetch=16,
        is_weight_positional=False, use_offsets=True, output_stride=-1, input_stride=-1,
        scale_bias_last=True, is_bf16_out=False, no_bag=False, output_bit_rate=-1, out_ty=FP32):
    """GenerateEmbeddingSpMDMNBitWithStrides (FbgemmEmbedding.h:151-174)."""
    if input_bit_rate not in (2, 4):
        raise ValueError("input_bit_rate must be 2 or 4")
    if is_bf16_out:
        out_ty = BF16
    if no_bag:
        # 4-bit rows copied to a 4-bit output is the one form the reference has
        # (src/RefImplementations.cc:1466-1474); it returns false for the others
        if input_bit_rate != 4 or output_bit_rate != 4:
            return lambda *args, **kwargs: False
        out_ty = INT4
    return _make_kernel(INT4 if input_bit_rate == 4 else INT2, block_size, normalize_by_lengths,
                        is_weight_positional, use_offsets, output_stride, input_stride,
                        scale_bias_last, out_ty, has_weight, False, no_bag)


def generate_embedding_spmdm_fp8_with_strides(
        block_size, normalize_by_lengths, is_weight_positional=False, use_offsets=True, output_stride=-1,
        input_stride=-1, exponent_bits=4, exponent_bias=7, is_bf16_out=False, out_ty=FP32):
    """GenerateEmbeddingSpMDMFP8WithStrides (FbgemmEmbedding.h:185-203): rows of 8-bit
    floats without scale/bias. The kernel takes ``weights`` as it comes (None = unweighted)."""
    if is_bf16_out:
        out_ty = BF16
    return _make_kernel(FP8, block_size, normalize_by_lengths, is_weight_positional, use_offsets, output_stride,
                        input_stride, True, out_ty, None, False, False, (exponent_bits, exponent_bias))


def generate_embedding_spmdm_nbit(bit_rate, block_size, has_weight, normalize_by_lengths, prefetch=16,
                                  is_weight_positional=False, use_offsets=True, out_ty=FP32):
    """GenerateEmbeddingSpMDMNBit (FbgemmEmbedding.h:124-140)."""
    return generate_embedding_spmdm_nbit_with_strides(
        bit_rate, block_size, has_weight, normalize_by_lengths, prefetch, is_weight_positional,
        use_offsets, out_ty=out_ty)


def generate_embedding_spmdm_rowwise_sparse(in_ty, block_size, has_weight, normalize_by_lengths,
                                            prefetch=16, is_weight_positional=False, use_offsets=True):
    """GenerateEmbeddingSpMDMRowWiseSparse (FbgemmEmbedding.h:229-243): the kernel
    takes ``compressed_indices_table`` as a trailing argument and writes fp32."""
    return _make_kernel(in_ty, block_size, normalize_by_lengths, is_weight_positional, use_offsets,
                        -1, -1, True, FP32, has_weight, True)


def generate_embedding_spmdm_nbit_rowwise_sparse(bit_rate, block_size, has_weight, normalize_by_lengths,
                                                 prefetch=16, is_weight_positional=False,
                                                 use_offsets=True):
    """GenerateEmbeddingSpMDMNBitRowWiseSparse (FbgemmEmbedding.h:250-262)."""
    if bit_rate not in (2, 4):
        raise ValueError("bit_rate must be 2 or 4")
    return _make_kernel(INT4 if bit_rate == 4 else INT2, block_size, normalize_by_lengths,
                        is_weight_positional, use_offsets, -1, -1, True, FP32, has_weight, True)


# ---- table-batched forward -------------------------------------------------


class TbePlan:
    """Owner of a fbgemm_amd_tbe_plan handle."""

    def __init__(self, weights_offsets, weights_tys, D_offsets, weights_placements,
                 dev_weights_bytes, uvm_weights_bytes, row_alignment):
        wo = weights_offsets.detach().to("cpu", torch.int64).contiguous()
        wt = weights_tys.detach().to("cpu", torch.uint8).contiguous()
        do = D_offsets.detach().to("cpu", torch.int32).contiguous()
        wp = weights_placements.detach().to("cpu", torch.int32).contiguous()
        self.T = do.numel() - 1
        self.total_D = int(do[-1])
        handle = C.c_void_p()
        check(_lib.lib().fbgemm_amd_tbe_plan_create(
            C.byref(handle), self.T, _ptr(wo), _ptr(wt), _ptr(do), _ptr(wp),
            dev_weights_bytes, uvm_weights_bytes, row_alignment))
        self.handle = handle

    def num_rows(self, t):
        return _lib.lib().fbgemm_amd_tbe_plan_num_rows(self.handle, t)

    def set_accumulate(self, mode):
        """ACC_EXACT (the reference's sequence of roundings, the default) or ACC_FAST (tolerance grade)."""
        check(_lib.lib().fbgemm_amd_tbe_plan_set_accumulate(self.handle, int(mode)))

    def set_index_remappings(self, index_remappings, index_remappings_offsets):
        """Build the compact form of order-preserving pruned-row mappings (2 bits per logical
        row) that the fused remap of the forward then uses whenever it is passed this very
        array. Made again when the array or its contents change (tensor version)."""
        if index_remappings is None or index_remappings.numel() == 0:
            check(_lib.lib().fbgemm_amd_tbe_plan_set_index_remappings(self.handle, None, 32, None, 0, _stream()))
            self._rank_key = None
            return 0
        ro = index_remappings_offsets.detach().to("cpu", torch.int64).contiguous()
        check(_lib.lib().fbgemm_amd_tbe_plan_set_index_remappings(
            self.handle, _ptr(index_remappings), _bits(index_remappings), _ptr(ro), ro.numel(), _stream()))
        self._rank_key = self.rank_key(index_remappings, index_remappings_offsets)
        self._rank_keepalive = (index_remappings, index_remappings_offsets)
        return self.rank_tables()

    @staticmethod
    def rank_key(index_remappings, index_remappings_offsets):
        """What the compact mappings were made from: the array and its offsets, by address and version."""
        return (index_remappings.data_ptr(), index_remappings._version, index_remappings.numel(),
                index_remappings_offsets.data_ptr(), index_remappings_offsets._version)

    def rank_tables(self):
        return _lib.lib().fbgemm_amd_tbe_plan_rank_tables(self.handle)

    def row_bytes(self, t):
        return _lib.lib().fbgemm_amd_tbe_plan_row_bytes(self.handle, t)

    def cached_work(self):
        """Work lists (one per batch size) the plan keeps."""
        return _lib.lib().fbgemm_amd_tbe_plan_cached_work(self.handle)

    def pinned_work(self):
        """How many of them a forward under stream capture has touched (a graph may hold them)."""
        return _lib.lib().fbgemm_amd_tbe_plan_pinned_work(self.handle)

    def trim(self):
        """Drop every cached work list, pinned ones included: graphs that contain forwards of this
        plan must be captured again afterwards."""
        check(_lib.lib().fbgemm_amd_tbe_plan_trim(self.handle))

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            try:
                _lib.lib().fbgemm_amd_tbe_plan_destroy(h)
            except Exception:
                pass


_plans = collections.OrderedDict()  # least recently used first
MAX_CACHED_PLANS = 64


def _plan_for(dev_weights, uvm_weights, weights_placements, weights_offsets, weights_tys, D_offsets,
              row_alignment):
    # The operator receives its metadata as device tensors on every call; the
    # host copy a plan needs is made once per distinct set of tensors.
    key = (weights_offsets.data_ptr(), weights_tys.data_ptr(), D_offsets.data_ptr(),
           weights_placements.data_ptr(), weights_offsets._version, D_offsets._version,
           weights_tys._version, weights_placements._version, D_offsets.numel(), dev_weights.numel(), uvm_weights.numel(),
           row_alignment)
    entry = _plans.get(key)
    if entry is None:
        plan = TbePlan(weights_offsets, weights_tys, D_offsets, weights_placements,
                       dev_weights.numel(), uvm_weights.numel(), row_alignment)
        if len(_plans) >= MAX_CACHED_PLANS:
            # the least recently used plan goes, but never one whose work lists a captured graph may hold
            # (a forward under stream capture pins them); when every plan is pinned the cache grows
            for old_key, (old, _) in _plans.items():
                if old.pinned_work() == 0:
                    del _plans[old_key]
                    break
        # the entry keeps the tensors alive: while it is cached their addresses cannot be handed to other tensors
        entry = _plans[key] = (plan, (weights_offsets, weights_tys, D_offsets, weights_placements))
    else:
        _plans.move_to_end(key)
    return entry[0]


def int_nbit_split_embedding_codegen_lookup_function(
        dev_weights, uvm_weights, weights_placements, weights_offsets, weights_tys, D_offsets,
        total_D, max_int2_D, max_int4_D, max_int8_D, max_float16_D, max_float32_D, indices,
        offsets, pooling_mode, indice_weights=None, output_dtype=FP16, lxu_cache_weights=None,
        lxu_cache_locations=None, row_alignment=None, max_float8_D=0, fp8_exponent_bits=-1,
        fp8_exponent_bias=-1, status=None, plan=None, index_remappings=None,
        index_remappings_offsets=None, accumulate=None):
    """Same arguments, in the same order, as the reference operator
    (embedding_forward_quantized_host_cpu.cpp:316-318). Returns [B, total_D].

    Input errors raise like the CPU operator does, unless ``status`` is given:
    then the call stays asynchronous and the caller reads the block later.

    ``index_remappings`` / ``index_remappings_offsets`` (the arguments of
    ``pruned_array_lookup``) fuse the pruned-row remap into the forward:
    ``indices`` are then logical ids.

    ``accumulate`` = ACC_EXACT / ACC_FAST sets the plan's arithmetic for this and
    later forwards (None leaves it as it is; a new plan is exact)."""
    _require_cuda(dev_weights, indices, offsets, indice_weights)
    if lxu_cache_locations is not None and lxu_cache_locations.numel() > 0:
        raise NotImplementedError("the LXU cache is not on this path: tables are resident in HBM")
    if offsets.dtype != indices.dtype:
        offsets = offsets.to(indices.dtype)  # as embedding_forward_quantized_host_cpu.cpp:111-113
    if pooling_mode == POOL_NONE:
        # embedding_forward_quantized_host_cpu.cpp:113-139: one row per index, unweighted, D = the largest max_*_D
        if row_alignment is None:
            row_alignment = 16
        if plan is None:
            plan = _plan_for(dev_weights, uvm_weights, weights_placements, weights_offsets, weights_tys,
                             D_offsets, row_alignment)
        D = max(max_int2_D, max_int4_D, max_int8_D, max_float16_D, max_float32_D, max_float8_D or 0)
        _set_fp8(plan, max_float8_D, fp8_exponent_bits, fp8_exponent_bias)
        total_L = indices.numel()
        if output_dtype in _OUT_TORCH:
            out = torch.empty((total_L, D), dtype=_OUT_TORCH[output_dtype], device=dev_weights.device)
        elif output_dtype in (INT8, INT4):
            out = torch.empty((total_L, D + 4 if output_dtype == INT8 else (D + 9) // 2), dtype=torch.uint8,
                              device=dev_weights.device)
        else:
            raise NotImplementedError(f"output_dtype {output_dtype} is not on this path")
        if total_L == 0 or (offsets.numel() - 1) // plan.T == 0:
            return out.zero_()
        own = status is None
        st = Status(dev_weights.device) if own else status
        check(_lib.lib().fbgemm_amd_tbe_forward_nobag(
            plan.handle, _ptr(dev_weights), _ptr(uvm_weights), _ptr(indices.contiguous()), _ptr(offsets.contiguous()),
            _bits(indices), indices.numel(), offsets.numel(), D, output_dtype, _ptr(out), _ptr(st.buf), _stream()))
        if own:
            bits, pos = st.read()
            if bits:
                _raise_embedding_error(bits, pos, indices, offsets, plan, (offsets.numel() - 1) // plan.T)
        return out
    if output_dtype not in _OUT_TORCH and output_dtype != INT8:
        raise NotImplementedError(f"output_dtype {output_dtype} is not on this path")
    if indice_weights is not None and indice_weights.numel() == 0:
        indice_weights = None
    if indice_weights is not None and indice_weights.dtype != torch.float32:
        indice_weights = indice_weights.float()  # embedding_forward_quantized_host.cpp:345
    if row_alignment is None:
        row_alignment = 16  # the GPU operator's default (embedding_forward_quantized_host.cpp:310)
    if plan is None:
        plan = _plan_for(dev_weights, uvm_weights, weights_placements, weights_offsets, weights_tys,
                         D_offsets, row_alignment)
    _set_fp8(plan, max_float8_D, fp8_exponent_bits, fp8_exponent_bias)
    if accumulate is not None:
        plan.set_accumulate(accumulate)
    T = plan.T
    if total_D != plan.total_D:
        raise ValueError(f"total_D {total_D} does not match D_offsets[-1] {plan.total_D}")
    B = (offsets.numel() - 1) // T
    if output_dtype == INT8:
        # every table's pooled vector quantized row-wise: D_t bytes, fp32 scale, fp32 bias (sparse_ops.py:571-577)
        out = torch.empty((B, total_D + 8 * T), dtype=torch.uint8, device=dev_weights.device)
    else:
        out = torch.empty((B, total_D), dtype=_OUT_TORCH[output_dtype], device=dev_weights.device)
    if B == 0:
        return out
    own = status is None
    st = Status(dev_weights.device) if own else status
    ro = None
    if index_remappings is not None:
        _require_cuda(index_remappings, index_remappings_offsets)
        if index_remappings_offsets.numel() != T + 1:
            raise ValueError(f"index_remappings_offsets holds {index_remappings_offsets.numel()} entries; the operator's "
                             f"{T} features need {T + 1} (one mapping slice per feature)")
        ro = index_remappings_offsets.to(torch.int64).contiguous()
        # the compact form of order-preserving mappings, made once per array and offsets (and again when either changes)
        key = TbePlan.rank_key(index_remappings, index_remappings_offsets)
        if getattr(plan, "_rank_key", None) != key:
            if torch.cuda.is_current_stream_capturing():
                # building the compact form allocates and synchronizes; and a mapping edited in place keeps its
                # address, so the forward would take the records made from the old contents into the graph
                if getattr(plan, "_rank_key", None) is not None:
                    raise RuntimeError("the pruned-row mappings changed since the plan's compact form of them was made: "
                                       "run one forward outside the stream capture after changing them")
            else:
                plan.set_index_remappings(index_remappings, index_remappings_offsets)
    check(_lib.lib().fbgemm_amd_tbe_forward_pruned(
        plan.handle, _ptr(dev_weights), _ptr(uvm_weights), _ptr(indices.contiguous()),
        _ptr(offsets.contiguous()), _bits(indices), indices.numel(), offsets.numel(), pooling_mode,
        _ptr(indice_weights), output_dtype, _ptr(out), _ptr(index_remappings),
        32 if index_remappings is None else _bits(index_remappings), _ptr(ro), 0 if ro is None else ro.numel(),
        _ptr(st.buf), _stream()))
    if own:
        bits, pos = st.read()
        if bits:
            _raise_embedding_error(bits, pos, indices, offsets, plan, B)
    return out


def _set_fp8(plan, max_float8_D, exponent_bits, exponent_bias):
    """FP8 tables need the operator's exponent bits and bias (check_fp8_params of the reference)."""
    if max_float8_D:
        if exponent_bits is None or exponent_bias is None or exponent_bits <= 0 or exponent_bias < 0:
            raise RuntimeError("FP8 tables need fp8_exponent_bits and fp8_exponent_bias")
        check(_lib.lib().fbgemm_amd_tbe_plan_set_fp8(plan.handle, exponent_bits, exponent_bias))


def _raise_embedding_error(bits, pos, indices, offsets, plan, B):
    # wording follows report_embedding_error (fbgemm_gpu/include/fbgemm_gpu/utils/cpu_utils.h:25-52)
    if bits & ERR_INDEX_OUT_OF_RANGE and pos >= 0:
        idx = int(indices[pos])
        off = offsets.cpu()
        t = int(torch.searchsorted(off[::B].contiguous(), torch.tensor([pos], dtype=off.dtype), right=True)) - 1
        t = max(0, min(plan.T - 1, t))
        raise RuntimeError(
            f"Index {pos} is out of bounds: {idx}, range 0 to {plan.num_rows(t)} (table {t})")
    raise RuntimeError(f"embedding lookup rejected its inputs (status bits {bits:#x})")


def pruned_array_lookup(indices, offsets, index_remappings, index_remappings_offsets):
    """pruned_array_lookup (embedding_forward_quantized_host_cpu.cpp:343-346)."""
    _require_cuda(indices, offsets, index_remappings, index_remappings_offsets)
    if indices.dtype != offsets.dtype:
        raise TypeError("indices and offsets must have the same dtype")
    T = index_remappings_offsets.numel() - 1
    dense = torch.empty_like(indices)
    ro = index_remappings_offsets.to(torch.int64).contiguous()
    check(_lib.lib().fbgemm_amd_pruned_array_lookup(
        _ptr(indices.contiguous()), _ptr(offsets.contiguous()), _bits(indices), offsets.numel(),
        _ptr(index_remappings), _bits(index_remappings), _ptr(ro), T, _ptr(dense), _stream()))
    return dense


def pruned_array_lookup_from_row_idx(update_row_indices, update_table_indices, index_remappings,
                                     index_remappings_offsets):
    """pruned_array_lookup_from_row_idx (embedding_inplace_update_cpu.cpp:199-251, schema :259-260): the
    logical rows of an update as physical rows; -1 for a pruned row."""
    _require_cuda(update_row_indices, update_table_indices, index_remappings, index_remappings_offsets)
    if update_table_indices.dtype != torch.int32:
        raise TypeError("update_table_indices must be int32")
    if update_table_indices.numel() != update_row_indices.numel():
        raise ValueError("update_table_indices and update_row_indices differ in length")
    T = index_remappings_offsets.numel() - 1
    dense = torch.empty_like(update_row_indices)
    ro = index_remappings_offsets.to(torch.int64).contiguous()
    check(_lib.lib().fbgemm_amd_pruned_array_lookup_from_row_idx(
        _ptr(update_row_indices.contiguous()), _bits(update_row_indices), _ptr(update_table_indices.contiguous()),
        update_row_indices.numel(), _ptr(index_remappings), _bits(index_remappings), _ptr(ro), T, _ptr(dense),
        _stream()))
    return dense


def emb_inplace_update(dev_weights, uvm_weights, weights_placements, weights_offsets, weights_tys, D_offsets,
                       update_weights, update_table_indices, update_row_indices, update_offsets, row_alignment=1,
                       lxu_cache_weights=None, lxu_cache_locations=None, status=None, plan=None):
    """emb_inplace_update (embedding_inplace_update_cpu.cpp:257-258): overwrites rows of the weights buffers
    in place. An update outside its table (or past ``update_weights``) raises unless ``status`` is given; a row id
    of -1 (a pruned row) is skipped."""
    _require_cuda(dev_weights, update_weights, update_table_indices, update_row_indices, update_offsets)
    if lxu_cache_locations is not None and lxu_cache_locations.numel() > 0:
        raise NotImplementedError("the LXU cache is not on this path: tables are resident in HBM")
    if update_weights.dtype != torch.uint8 or update_table_indices.dtype != torch.int32 or update_offsets.dtype != torch.int64:
        raise TypeError("update_weights is uint8, update_table_indices int32, update_offsets int64")
    n = update_row_indices.numel()
    if update_table_indices.numel() != n or update_offsets.numel() < n:
        raise ValueError("update_table_indices / update_offsets do not cover update_row_indices")
    if n == 0:
        return
    if plan is None:
        plan = _plan_for(dev_weights, uvm_weights, weights_placements, weights_offsets, weights_tys, D_offsets,
                         row_alignment)
    own = status is None
    st = Status(dev_weights.device) if own else status
    update_weights = update_weights.contiguous()
    check(_lib.lib().fbgemm_amd_tbe_inplace_update(
        plan.handle, _ptr(dev_weights), _ptr(uvm_weights), _ptr(update_weights), update_weights.numel(),
        _ptr(update_table_indices.contiguous()), _ptr(update_row_indices.contiguous()), _bits(update_row_indices),
        _ptr(update_offsets.contiguous()), n, _ptr(st.buf), _stream()))
    if own:
        bits, pos = st.read()
        if bits & ERR_INDEX_OUT_OF_RANGE:
            raise RuntimeError(f"update {pos} names table {int(update_table_indices[pos])}, row "
                               f"{int(update_row_indices[pos])}, which does not exist")
        if bits:
            raise RuntimeError("an update reads past the end of update_weights")


def padded_row_size_in_bytes(dim, weight_ty, row_alignment, scale_bias_bytes=4):
    """nbit::padded_row_size_in_bytes (embedding_common.h:217-225)."""
    return _lib.lib().fbgemm_amd_padded_row_size_in_bytes(dim, weight_ty, row_alignment, scale_bias_bytes)


def unpadded_row_size_in_bytes(dim, weight_ty, scale_bias_bytes=4):
    """nbit::unpadded_row_size_in_bytes (embedding_common.h:189-215)."""
    return _lib.lib().fbgemm_amd_unpadded_row_size_in_bytes(dim, weight_ty, scale_bias_bytes)


BOUNDS_FATAL, BOUNDS_WARNING, BOUNDS_IGNORE = 0, 1, 2


def bounds_check_indices(rows_per_table, indices, offsets, bounds_check_mode, warning, weights=None,
                         B_offsets=None, max_B=-1):
    """bounds_check_indices (fbgemm_gpu/codegen/utils/embedding_bounds_check_host_cpu.cpp:76-219,
    schema :240-256): in place on ``indices`` / ``offsets`` / ``warning``.

    FATAL raises where the reference's CPU operator raises (after a
    synchronization); WARNING and IGNORE repair and stay asynchronous."""
    _require_cuda(rows_per_table, indices, offsets, warning, weights, B_offsets)
    if indices.dtype != offsets.dtype:
        raise TypeError("indices and offsets must have the same dtype")
    if not (indices.is_contiguous() and offsets.is_contiguous()):
        raise ValueError("indices and offsets are modified in place and must be contiguous")
    if weights is not None and weights.numel() != 0 and weights.size(0) != indices.numel():
        raise RuntimeError(f"weights size {weights.size(0)} is not equal to indices size {indices.numel()}")
    if B_offsets is not None and max_B < 0:
        raise RuntimeError("max_B must not be negative with B_offsets")
    rpt = rows_per_table.to(torch.int64).contiguous()
    bo = None if B_offsets is None else B_offsets.to(torch.int32).contiguous()
    status = Status(indices.device) if bounds_check_mode == BOUNDS_FATAL else None
    check(_lib.lib().fbgemm_amd_bounds_check_indices(
        _ptr(rpt), rpt.numel(), _ptr(indices), _ptr(offsets), _bits(indices), indices.numel(), offsets.numel(),
        int(bounds_check_mode), _ptr(warning), _ptr(bo), None if status is None else _ptr(status.buf), _stream()))
    if status is not None:
        bits, pos = status.read()
        if bits & ERR_LENGTH_MISMATCH:
            raise RuntimeError(f"the last offset is not the number of indices ({indices.numel()})")
        if bits & ERR_BAG_OVERRUN:
            raise RuntimeError("offsets are negative, decreasing or beyond the number of indices")
        if bits & ERR_INDEX_OUT_OF_RANGE:
            raise RuntimeError(f"Index {pos} is out of bounds: {int(indices[pos])}")


def pruned_hashmap_lookup(indices, offsets, hash_table, hash_table_offsets):
    """pruned_hashmap_lookup (embedding_forward_quantized_host_cpu.cpp:338-341;
    embedding_forward_quantized_cpu_template.cpp:524-603)."""
    _require_cuda(indices, offsets, hash_table, hash_table_offsets)
    if indices.dtype != offsets.dtype:
        raise TypeError("indices and offsets must have the same dtype")
    T = hash_table_offsets.numel() - 1
    if T <= 0 or (offsets.numel() - 1) // T <= 0:
        raise RuntimeError("pruned_hashmap_lookup needs B > 0")  # TORCH_CHECK(B > 0), :537
    dense = torch.empty_like(indices)
    hto = hash_table_offsets.to(torch.int64).contiguous()
    check(_lib.lib().fbgemm_amd_pruned_hashmap_lookup(
        _ptr(indices.contiguous()), _ptr(offsets.contiguous()), _bits(indices), offsets.numel(),
        _ptr(hash_table.contiguous()), _bits(hash_table), _ptr(hto), T, _ptr(dense), _stream()))
    return dense


QLAYOUT_TRAILER, QLAYOUT_TBE = 0, 1


def quantized_row_bytes(cols, bit_rate, sb_float=False, layout=QLAYOUT_TRAILER):
    epb = 8 // bit_rate
    return (cols + epb - 1) // epb + (8 if (sb_float and layout == QLAYOUT_TRAILER) else 4)


def quantize_rowwise(input, bit_rate, sb_float=False, layout=QLAYOUT_TRAILER, out=None, rowwise_min_max=None):
    """fp32 / fp16 ``[rows, cols]`` -> fused quantized rows, uint8 ``[rows, stride]``
    (FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf, src/QuantUtils.cc:534-611;
    FloatOrHalfToFused8BitRowwiseQuantizedSBFloat, :677-718; TBE re-layout as
    fbgemm_gpu/fbgemm_gpu/tbe/utils/quantize.py:47-70). ``out`` may be a wider
    (padded) row buffer; bytes beyond the row's own are left alone.
    ``rowwise_min_max`` (``[rows, 2]``, the input's dtype: minimum, maximum) takes the
    place of each row's own extremes (src/QuantUtilsAvx2.cc:1605-1628, :1831-1853)."""
    _require_cuda(input, out, rowwise_min_max)
    if input.dim() != 2 or input.dtype not in (torch.float32, torch.float16):
        raise TypeError("input must be a 2-D fp32 or fp16 tensor")
    input = input.contiguous()
    rows, cols = input.shape
    if out is None:
        out = torch.empty((rows, quantized_row_bytes(cols, bit_rate, sb_float, layout)), dtype=torch.uint8,
                          device=input.device)
    if out.dtype != torch.uint8 or out.dim() != 2 or out.size(0) != rows or out.stride(1) != 1:
        raise ValueError("out must be uint8 [rows, stride] with unit column stride")
    if rowwise_min_max is not None:
        if rowwise_min_max.dtype != input.dtype or tuple(rowwise_min_max.shape) != (rows, 2):
            raise ValueError("rowwise_min_max must be [rows, 2] of the input's dtype")
        rowwise_min_max = rowwise_min_max.contiguous()
    check(_lib.lib().fbgemm_amd_quantize_rowwise_min_max(
        _ptr(input), _TORCH_OUT[input.dtype], rows, cols, bit_rate, int(sb_float), layout,
        out.stride(0) if rows > 1 else out.size(1), _ptr(out),
        _ptr(rowwise_min_max) if rowwise_min_max is not None else None, _stream()))
    return out


def dequantize_rowwise(input, cols, bit_rate, sb_float=False, layout=QLAYOUT_TRAILER, output_dtype=torch.float32):
    """Fused quantized rows uint8 ``[rows, stride]`` -> ``[rows, cols]`` fp32 / fp16 / bf16
    (FusedNBitRowwiseQuantizedSBHalfToFloatOrHalf, src/QuantUtils.cc:743-789;
    Fused8BitRowwiseQuantizedSBFloatToFloatOrHalf, :847-892)."""
    _require_cuda(input)
    if input.dtype != torch.uint8 or input.dim() != 2 or input.stride(1) != 1:
        raise ValueError("input must be uint8 [rows, stride] with unit column stride")
    rows = input.size(0)
    out = torch.empty((rows, cols), dtype=output_dtype, device=input.device)
    check(_lib.lib().fbgemm_amd_dequantize_rowwise(
        _ptr(input), rows, input.stride(0) if rows > 1 else input.size(1), cols, bit_rate, int(sb_float), layout,
        _TORCH_OUT[output_dtype], _ptr(out), _stream()))
    return out


def float_to_hfp8_quantized(input, ebits, exponent_bias, max_pos):
    """FloatToHFP8Quantized (fbgemm_gpu/src/quantize_ops/quantize_ops_cpu.cpp:571-594):
    fp32 ``[rows, cols]`` -> hfp8 codes, uint8, same shape."""
    _require_cuda(input)
    if input.dtype != torch.float32 or input.dim() != 2:
        raise ValueError("input must be a 2-d float32 tensor")
    input = input.contiguous()
    out = torch.empty(input.shape, dtype=torch.uint8, device=input.device)
    check(_lib.lib().fbgemm_amd_float_to_hfp8(_ptr(input), input.numel(), ebits, exponent_bias, float(max_pos), _ptr(out), _stream()))
    return out


def hfp8_quantized_to_float(input, ebits, exponent_bias):
    """HFP8QuantizedToFloat (quantize_ops_cpu.cpp:596-620): hfp8 codes ``[rows, cols]`` -> fp32."""
    _require_cuda(input)
    if input.dtype != torch.uint8 or input.dim() != 2:
        raise ValueError("input must be a 2-d uint8 tensor")
    input = input.contiguous()
    out = torch.empty(input.shape, dtype=torch.float32, device=input.device)
    check(_lib.lib().fbgemm_amd_hfp8_to_float(_ptr(input), input.numel(), ebits, exponent_bias, _ptr(out), _stream()))
    return out


def compressed_indices_remap(indices, compressed_indices_mapping, offsets, weights=None):
    """fbgemm::compressed_indices_remap (FbgemmEmbedding.h:392-401; src/RefImplementations.cc:2308-2333):
    drops the entries of pruned rows, maps the others to physical rows, rewrites offsets (and weights).
    Returns (out_indices, out_offsets, out_weights or None); the outputs have the inputs' sizes, their
    first out_offsets[-1] entries are meaningful. Raises on an index outside the mapping."""
    _require_cuda(indices, compressed_indices_mapping, offsets, weights)
    if indices.dtype != offsets.dtype:
        raise TypeError("indices and offsets must have the same dtype")
    if compressed_indices_mapping.dtype != torch.int32:
        raise TypeError("compressed_indices_mapping must be int32")
    if weights is not None and weights.dtype != torch.float32:
        raise TypeError("weights must be float32")
    indices, offsets, mapping = indices.contiguous(), offsets.contiguous(), compressed_indices_mapping.contiguous()
    out_indices = torch.empty_like(indices)
    out_offsets = torch.empty_like(offsets)
    out_weights = None if weights is None else torch.empty_like(weights)
    st = Status(indices.device)
    check(_lib.lib().fbgemm_amd_compressed_indices_remap(
        offsets.numel(), _ptr(indices), _bits(indices), _ptr(mapping), mapping.numel(), _ptr(offsets),
        _ptr(None if weights is None else weights.contiguous()), _ptr(out_indices), _ptr(out_offsets), _ptr(out_weights),
        _ptr(st.buf), _stream()))
    bits, pos = st.read()
    if bits:
        raise IndexError(f"compressed_indices_remap: index at position {pos} is outside the mapping")
    return out_indices, out_offsets, out_weights


def embedding_bag_rowwise_prune(weight, indicator, threshold, compressed_indices_dtype, abs=True, min_num_rows=0,
                                min_save_ratio=1.0):
    """embedding_bag_rowwise_prune (fbgemm_gpu/src/sparse_ops/sparse_ops_cpu.cpp:2836-2893), on the GPU:
    keeps the rows of ``weight`` whose ``indicator`` exceeds ``threshold`` (and the last rows needed to
    reach ``min_num_rows``); returns (kept rows, remap) with remap[i] the new row id or -1. When
    pruning would not save memory (``min_save_ratio``) the weights come back whole with the map [0]."""
    _require_cuda(weight, indicator)
    if weight.dim() != 2:
        raise ValueError("Tensor 'weights' must have 2 dimension(s)")
    if indicator.numel() != weight.size(0):
        raise ValueError("Number of elements in 'indicator' should be equivalent to number of rows in 'weights'.")
    if not threshold >= 0.0:
        raise ValueError("Threshold should be greater than or equal to zero.")
    if compressed_indices_dtype not in (torch.int32, torch.int64):
        raise ValueError("'compressed_indices_dtype' should be Int/Long.")
    rows, cols = weight.shape
    if min_save_ratio is not None:
        # should_prune (sparse_ops_cpu.cpp:2773-2794): sized as fp32 rows plus a 4-byte map entry per
        # original row, with min_num_rows standing for the rows that stay
        if not rows * 4 + min_num_rows * cols * 4 < min_save_ratio * 4 * rows * cols:
            return weight, torch.zeros(1, dtype=compressed_indices_dtype, device=weight.device)
    weight = weight.contiguous()
    indicator = indicator.to(torch.float32).contiguous()
    remap = torch.empty(rows, dtype=compressed_indices_dtype, device=weight.device)
    kept = C.c_int64(0)
    check(_lib.lib().fbgemm_amd_rowwise_prune_map(_ptr(indicator), rows, float(threshold), int(bool(abs)), int(min_num_rows),
                                                  _bits(remap), _ptr(remap), C.byref(kept), _stream()))
    out = torch.empty((kept.value, cols), dtype=weight.dtype, device=weight.device)
    check(_lib.lib().fbgemm_amd_rowwise_prune_gather(_ptr(weight), rows, cols * weight.element_size(), _ptr(remap),
                                                     _bits(remap), _ptr(out), kept.value, _stream()))
    return out, remap


def pruned_hashmap_insert(indices, dense_indices, offsets, hash_table, hash_table_offsets):
    """pruned_hashmap_insert (embedding_forward_quantized_host_cpu.cpp:331-334;
    embedding_forward_quantized_cpu_template.cpp:124-201): HOST tensors, in place
    on ``hash_table`` ([slots, 2], -1 = empty), as in the reference, whose GPU
    module builds the map on the CPU too."""
    for t in (indices, dense_indices, offsets, hash_table, hash_table_offsets):
        if t.is_cuda:
            raise ValueError("pruned_hashmap_insert works on host tensors")
    if indices.dtype != offsets.dtype:
        raise TypeError("indices and offsets must have the same dtype")
    if not hash_table.is_contiguous() or hash_table.dim() != 2 or hash_table.size(1) != 2:
        raise ValueError("hash_table must be a contiguous [slots, 2] tensor")
    indices = indices.contiguous()
    dense = dense_indices.to(indices.dtype).contiguous()
    offsets = offsets.contiguous()
    hto = hash_table_offsets.to(torch.int64).contiguous()
    check(_lib.lib().fbgemm_amd_pruned_hashmap_insert_host(
        _ptr(indices), _ptr(dense), _ptr(offsets), _bits(indices), offsets.numel(), _ptr(hash_table),
        _bits(hash_table), _ptr(hto), hto.numel() - 1))
