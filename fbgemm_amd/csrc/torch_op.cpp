// torch operator registration: the reference's schema strings, verbatim, with
// the HIP library behind the CUDA dispatch key (which is what HIP devices use
// in PyTorch). Reference: TORCH_LIBRARY_FRAGMENT(fbgemm, ...) in
// fbgemm_gpu/codegen/inference/embedding_forward_quantized_host_cpu.cpp:310-347
// and the GPU dispatcher embedding_forward_quantized_host.cpp:259-370,574-583.
//
// torch is used for what it owns: tensors (HBM) and the current stream. All
// work goes through the C ABI of include/fbgemm_amd.h.
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <algorithm>
#include <map>
#include <memory>
#include <mutex>
#include <tuple>

#include "../../include/fbgemm_amd.h"
#include "cache_policy.h"

namespace {

using at::Tensor;

void* current_stream(const Tensor& t) {
  return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

// One plan per distinct set of metadata tensors (the operator receives them as
// device tensors on every call; the host copy a plan needs is made once).
// A plan is cached per set of metadata tensors: their addresses AND versions (an in-place edit of
// weights_offsets / weights_tys / D_offsets makes a new plan), sizes and the row alignment.
struct PlanKey {
  const void *wo, *wt, *dofs, *wp;
  int64_t v_wo, v_wt, v_dofs, v_wp;
  int64_t T, dev_bytes, uvm_bytes, row_alignment;
  bool operator<(const PlanKey& o) const {
    return std::tie(wo, wt, dofs, wp, v_wo, v_wt, v_dofs, v_wp, T, dev_bytes, uvm_bytes, row_alignment) <
        std::tie(o.wo, o.wt, o.dofs, o.wp, o.v_wo, o.v_wt, o.v_dofs, o.v_wp, o.T, o.dev_bytes, o.uvm_bytes, o.row_alignment);
  }
};
// Owner of a plan handle. Forwards hold a reference while they launch, so a plan that the cache
// drops is destroyed only after the last of them has returned (the destructor waits for the device).
struct PlanHolder {
  fbgemm_amd_tbe_plan* plan = nullptr;
  Tensor keep[4]; // the key's tensors: alive while cached, so their addresses are not handed to other tensors
  ~PlanHolder() { fbgemm_amd_tbe_plan_destroy(plan); }
};
struct PlanEntry {
  std::shared_ptr<PlanHolder> holder;
  uint64_t last_use;
};
constexpr size_t MAX_CACHED_PLANS = 64; // beyond: the least recently used plan that no graph can hold goes
std::mutex g_mu;                        // guards the two maps below, never held across a launch
std::map<PlanKey, PlanEntry> g_plans;
uint64_t g_use_clock = 0;
std::map<int, Tensor> g_status; // one status block per device, never freed

Tensor status_block(const Tensor& like) {
  const int dev = like.device().index();
  std::lock_guard<std::mutex> lk(g_mu);
  auto it = g_status.find(dev);
  if (it == g_status.end()) {
    Tensor st = at::zeros({4}, like.options().dtype(at::kInt));
    TORCH_CHECK(fbgemm_amd_status_clear(st.data_ptr(), current_stream(like)) == 0, fbgemm_amd_last_error());
    it = g_status.emplace(dev, st).first;
  }
  return it->second;
}

std::shared_ptr<PlanHolder> plan_for(const Tensor& dev_weights, const Tensor& uvm_weights, const Tensor& placements,
                                     const Tensor& weights_offsets, const Tensor& weights_tys, const Tensor& D_offsets,
                                     int64_t row_alignment) {
  const PlanKey key{weights_offsets.data_ptr(), weights_tys.data_ptr(), D_offsets.data_ptr(), placements.data_ptr(),
                    (int64_t)weights_offsets._version(), (int64_t)weights_tys._version(), (int64_t)D_offsets._version(),
                    (int64_t)placements._version(), D_offsets.numel() - 1, dev_weights.numel(), uvm_weights.numel(),
                    row_alignment};
  {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_plans.find(key);
    if (it != g_plans.end()) {
      it->second.last_use = ++g_use_clock;
      return it->second.holder;
    }
  }
  const Tensor wo = weights_offsets.to(at::kCPU, at::kLong).contiguous();
  const Tensor wt = weights_tys.to(at::kCPU, at::kByte).contiguous();
  const Tensor dofs = D_offsets.to(at::kCPU, at::kInt).contiguous();
  const Tensor wp = placements.to(at::kCPU, at::kInt).contiguous();
  auto holder = std::make_shared<PlanHolder>();
  const int rc = fbgemm_amd_tbe_plan_create(
      &holder->plan, (int32_t)(dofs.numel() - 1), wo.data_ptr<int64_t>(), wt.data_ptr<uint8_t>(), dofs.data_ptr<int32_t>(),
      wp.data_ptr<int32_t>(), dev_weights.numel(), uvm_weights.numel(), row_alignment);
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  holder->keep[0] = weights_offsets;
  holder->keep[1] = weights_tys;
  holder->keep[2] = D_offsets;
  holder->keep[3] = placements;
  std::shared_ptr<PlanHolder> evicted; // destroyed (device synchronize) after the lock is released
  {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_plans.find(key); // another thread may have made the same plan meanwhile
    if (it != g_plans.end()) {
      it->second.last_use = ++g_use_clock;
      return it->second.holder;
    }
    if (g_plans.size() >= MAX_CACHED_PLANS) {
      // the least recently used plan that no captured graph can hold (a forward under stream
      // capture pins what it touches); when every plan is pinned the cache grows instead
      auto victim = fbgemm_amd::least_recently_used_not_held(
          g_plans, [](const PlanEntry& e) { return fbgemm_amd_tbe_plan_pinned_work(e.holder->plan) != 0; },
          [](const PlanEntry& e) { return e.last_use; });
      if (victim != g_plans.end()) {
        evicted = victim->second.holder;
        g_plans.erase(victim);
      }
    }
    g_plans.emplace(key, PlanEntry{holder, ++g_use_clock});
  }
  return holder;
}

at::ScalarType out_scalar_type(int64_t output_dtype) {
  switch (output_dtype) {
    case FBGEMM_AMD_FP32: return at::kFloat;
    case FBGEMM_AMD_FP16: return at::kHalf;
    case FBGEMM_AMD_BF16: return at::kBFloat16;
    default: TORCH_CHECK(false, "fbgemm_amd: output_dtype ", output_dtype, " (int8 / int4 outputs) is not on this path");
  }
}

Tensor int_nbit_split_embedding_codegen_lookup_function_hip(
    Tensor dev_weights, Tensor uvm_weights, Tensor weights_placements, Tensor weights_offsets, Tensor weights_tys,
    Tensor D_offsets, int64_t total_D, int64_t max_int2_D, int64_t max_int4_D, int64_t max_int8_D,
    int64_t max_float16_D, int64_t max_float32_D, Tensor indices, Tensor offsets, int64_t pooling_mode,
    std::optional<Tensor> indice_weights, int64_t output_dtype, std::optional<Tensor> /*lxu_cache_weights*/,
    std::optional<Tensor> lxu_cache_locations, std::optional<int64_t> row_alignment,
    std::optional<int64_t> max_float8_D, std::optional<int64_t> fp8_exponent_bits,
    std::optional<int64_t> fp8_exponent_bias) {
  TORCH_CHECK(dev_weights.is_cuda() && indices.is_cuda() && offsets.is_cuda(), "fbgemm_amd: tensors must be on the GPU");
  TORCH_CHECK(pooling_mode == FBGEMM_AMD_POOL_SUM || pooling_mode == FBGEMM_AMD_POOL_MEAN || pooling_mode == FBGEMM_AMD_POOL_NONE,
              "fbgemm_amd: unknown pooling mode ", pooling_mode);
  TORCH_CHECK(!lxu_cache_locations || lxu_cache_locations->numel() == 0,
              "fbgemm_amd: the LXU cache is not on this path (tables are resident in HBM)");
  TORCH_CHECK(indices.scalar_type() == at::kInt || indices.scalar_type() == at::kLong, "indices must be int32 or int64");
  // embedding_forward_quantized_host_cpu.cpp:111-113
  if (offsets.scalar_type() != indices.scalar_type()) offsets = offsets.to(indices.scalar_type());
  indices = indices.contiguous();
  offsets = offsets.contiguous();
  Tensor w;
  if (indice_weights && indice_weights->numel() > 0) {
    w = indice_weights->to(at::kFloat).contiguous(); // embedding_forward_quantized_host.cpp:345
  }
  const int64_t align = row_alignment ? *row_alignment : 16; // embedding_forward_quantized_host.cpp:310
  const std::shared_ptr<PlanHolder> holder = plan_for(dev_weights, uvm_weights, weights_placements, weights_offsets,
                                                      weights_tys, D_offsets, align);
  fbgemm_amd_tbe_plan* plan = holder->plan;
  if (max_float8_D && *max_float8_D > 0) {
    TORCH_CHECK(fp8_exponent_bits && fp8_exponent_bias && *fp8_exponent_bits > 0 && *fp8_exponent_bias >= 0,
                "FP8 tables need fp8_exponent_bits and fp8_exponent_bias");
    TORCH_CHECK(fbgemm_amd_tbe_plan_set_fp8(plan, (int32_t)*fp8_exponent_bits, (int32_t)*fp8_exponent_bias) == 0,
                "fbgemm_amd: ", fbgemm_amd_last_error());
  }
  const int64_t T = D_offsets.numel() - 1;
  TORCH_CHECK(T > 0 && total_D > 0);
  const int64_t B = (offsets.numel() - 1) / T;
  TORCH_CHECK(B >= 0);
  if (pooling_mode == FBGEMM_AMD_POOL_NONE) {
    // embedding_forward_quantized_host_cpu.cpp:113-139: one row per index, D = the largest max_*_D
    const int64_t D = std::max({max_int2_D, max_int4_D, max_int8_D, max_float16_D, max_float32_D, max_float8_D.value_or(0)});
    const int64_t total_L = indices.numel();
    Tensor out;
    if (output_dtype == FBGEMM_AMD_INT8 || output_dtype == FBGEMM_AMD_INT4)
      out = at::empty({total_L, output_dtype == FBGEMM_AMD_INT8 ? D + 4 : (D + 9) / 2}, dev_weights.options().dtype(at::kByte));
    else
      out = at::empty({total_L, D}, dev_weights.options().dtype(out_scalar_type(output_dtype)));
    if (total_L == 0 || B == 0) return out.zero_();
    Tensor st = status_block(dev_weights);
    const int rc = fbgemm_amd_tbe_forward_nobag(
        plan, dev_weights.data_ptr(), uvm_weights.numel() ? uvm_weights.data_ptr() : nullptr, indices.data_ptr(),
        offsets.data_ptr(), indices.scalar_type() == at::kLong ? 64 : 32, indices.numel(), offsets.numel(), (int32_t)D,
        (int32_t)output_dtype, out.data_ptr(), st.data_ptr(), current_stream(dev_weights));
    TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
    return out;
  }
  // 8-bit output: every table's pooled vector quantized row-wise, D_t bytes + fp32 scale + fp32 bias
  // (fbgemm_gpu/fbgemm_gpu/sparse_ops.py:571-577)
  Tensor out = output_dtype == FBGEMM_AMD_INT8
      ? at::empty({B, total_D + 8 * T}, dev_weights.options().dtype(at::kByte))
      : at::empty({B, total_D}, dev_weights.options().dtype(out_scalar_type(output_dtype)));
  if (B == 0) return out;
  Tensor st = status_block(dev_weights);
  const int rc = fbgemm_amd_tbe_forward(
      plan, dev_weights.data_ptr(), uvm_weights.numel() ? uvm_weights.data_ptr() : nullptr, indices.data_ptr(),
      offsets.data_ptr(), indices.scalar_type() == at::kLong ? 64 : 32, indices.numel(), offsets.numel(),
      (int32_t)pooling_mode, w.defined() ? w.data_ptr<float>() : nullptr, (int32_t)output_dtype, out.data_ptr(),
      st.data_ptr(), current_stream(dev_weights));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  return out;
}

// The operator the reference's module calls when it owns a UVM cache
// (embedding_forward_quantized_host_cpu.cpp:323-329): the same forward. Here
// every table is resident in HBM, so the cache arguments must be absent.
Tensor int_nbit_split_embedding_uvm_caching_codegen_lookup_function_hip(
    Tensor dev_weights, Tensor uvm_weights, Tensor weights_placements, Tensor weights_offsets, Tensor weights_tys,
    Tensor D_offsets, int64_t total_D, int64_t max_int2_D, int64_t max_int4_D, int64_t max_int8_D,
    int64_t max_float16_D, int64_t max_float32_D, Tensor indices, Tensor offsets, int64_t pooling_mode,
    std::optional<Tensor> indice_weights, int64_t output_dtype, std::optional<Tensor> lxu_cache_weights,
    std::optional<Tensor> lxu_cache_locations, std::optional<int64_t> row_alignment,
    std::optional<int64_t> max_float8_D, std::optional<int64_t> fp8_exponent_bits,
    std::optional<int64_t> fp8_exponent_bias, std::optional<Tensor> cache_hash_size_cumsum,
    std::optional<int64_t> total_cache_hash_size, std::optional<Tensor> /*cache_index_table_map*/,
    std::optional<Tensor> /*lxu_cache_state*/, std::optional<Tensor> /*lxu_state*/) {
  TORCH_CHECK((!cache_hash_size_cumsum || cache_hash_size_cumsum->numel() == 0) &&
                  (!total_cache_hash_size || *total_cache_hash_size <= 0),
              "fbgemm_amd: the UVM cache is not on this path (tables are resident in HBM)");
  return int_nbit_split_embedding_codegen_lookup_function_hip(
      std::move(dev_weights), std::move(uvm_weights), std::move(weights_placements), std::move(weights_offsets),
      std::move(weights_tys), std::move(D_offsets), total_D, max_int2_D, max_int4_D, max_int8_D, max_float16_D,
      max_float32_D, std::move(indices), std::move(offsets), pooling_mode, std::move(indice_weights), output_dtype,
      std::move(lxu_cache_weights), std::move(lxu_cache_locations), row_alignment.value_or(-1) > 0 ? row_alignment : std::nullopt,
      max_float8_D, fp8_exponent_bits, fp8_exponent_bias);
}

// Out-of-range indices are recorded on the device and do not stop the stream
// (the reference's GPU operator does not look at them at all; its CPU operator
// raises). This reads the record: synchronizes, returns the FBGEMM_AMD_ERR_*
// bits seen since the last call and clears them.
int64_t lookup_status(Tensor like) {
  Tensor st = status_block(like);
  int32_t bits = 0;
  int64_t pos = -1;
  TORCH_CHECK(fbgemm_amd_status_read(st.data_ptr(), current_stream(like), &bits, &pos) == 0, fbgemm_amd_last_error());
  TORCH_CHECK(fbgemm_amd_status_clear(st.data_ptr(), current_stream(like)) == 0, fbgemm_amd_last_error());
  return bits;
}

Tensor pruned_array_lookup_hip(Tensor indices, Tensor offsets, Tensor index_remappings, Tensor index_remappings_offsets) {
  TORCH_CHECK(indices.is_cuda() && offsets.is_cuda() && index_remappings.is_cuda() && index_remappings_offsets.is_cuda());
  TORCH_CHECK(indices.scalar_type() == offsets.scalar_type(), "indices and offsets must have the same dtype");
  indices = indices.contiguous();
  offsets = offsets.contiguous();
  index_remappings = index_remappings.contiguous();
  const Tensor ro = index_remappings_offsets.to(at::kLong).contiguous();
  const int64_t T = ro.numel() - 1;
  Tensor dense = at::empty_like(indices);
  const int rc = fbgemm_amd_pruned_array_lookup(
      indices.data_ptr(), offsets.data_ptr(), indices.scalar_type() == at::kLong ? 64 : 32, offsets.numel(),
      index_remappings.data_ptr(), index_remappings.scalar_type() == at::kLong ? 64 : 32, ro.data_ptr<int64_t>(),
      (int32_t)T, dense.data_ptr(), current_stream(indices));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  return dense;
}

// pruned_array_lookup_from_row_idx (fbgemm_gpu/src/embedding_inplace_ops/embedding_inplace_update_cpu.cpp:199-251)
Tensor pruned_array_lookup_from_row_idx_hip(const Tensor& update_row_indices, const Tensor& update_table_indices,
                                            const Tensor& index_remappings, const Tensor& index_remappings_offsets) {
  TORCH_CHECK(update_row_indices.is_cuda() && update_table_indices.is_cuda() && index_remappings.is_cuda() &&
              index_remappings_offsets.is_cuda());
  TORCH_CHECK(update_table_indices.scalar_type() == at::kInt, "update_table_indices must be int32");
  TORCH_CHECK(update_table_indices.numel() == update_row_indices.numel());
  const Tensor rows = update_row_indices.contiguous();
  const Tensor tables = update_table_indices.contiguous();
  const Tensor remap = index_remappings.contiguous();
  const Tensor ro = index_remappings_offsets.to(at::kLong).contiguous();
  Tensor dense = at::empty_like(rows);
  const int rc = fbgemm_amd_pruned_array_lookup_from_row_idx(
      rows.data_ptr(), rows.scalar_type() == at::kLong ? 64 : 32, tables.data_ptr<int32_t>(), rows.numel(),
      remap.data_ptr(), remap.scalar_type() == at::kLong ? 64 : 32, ro.data_ptr<int64_t>(), (int32_t)(ro.numel() - 1),
      dense.data_ptr(), current_stream(rows));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  return dense;
}

// emb_inplace_update (embedding_inplace_update_cpu.cpp:72-120): rows of the weights buffers are overwritten in
// place. Updates that name no row are skipped and recorded where lookup_status reads them.
void emb_inplace_update_hip(Tensor dev_weights, Tensor uvm_weights, Tensor weights_placements, Tensor weights_offsets,
                            Tensor weights_tys, Tensor D_offsets, Tensor update_weights, Tensor update_table_idx,
                            Tensor update_row_idx, Tensor update_offsets, const int64_t row_alignment,
                            std::optional<Tensor> /*lxu_cache_weights*/, std::optional<Tensor> lxu_cache_locations) {
  TORCH_CHECK(dev_weights.is_cuda() && update_weights.is_cuda() && update_table_idx.is_cuda() && update_row_idx.is_cuda() &&
                  update_offsets.is_cuda(), "fbgemm_amd: tensors must be on the GPU");
  TORCH_CHECK(!lxu_cache_locations || lxu_cache_locations->numel() == 0,
              "fbgemm_amd: the LXU cache is not on this path (tables are resident in HBM)");
  TORCH_CHECK(update_weights.scalar_type() == at::kByte && update_table_idx.scalar_type() == at::kInt &&
              update_offsets.scalar_type() == at::kLong, "update_weights is uint8, update_table_indices int32, update_offsets int64");
  const int64_t n = update_row_idx.numel();
  TORCH_CHECK(update_table_idx.numel() == n && update_offsets.numel() >= n);
  if (n == 0) return;
  update_weights = update_weights.contiguous();
  update_table_idx = update_table_idx.contiguous();
  update_row_idx = update_row_idx.contiguous();
  update_offsets = update_offsets.contiguous();
  const std::shared_ptr<PlanHolder> holder = plan_for(dev_weights, uvm_weights, weights_placements, weights_offsets,
                                                      weights_tys, D_offsets, row_alignment);
  fbgemm_amd_tbe_plan* plan = holder->plan;
  Tensor st = status_block(dev_weights);
  const int rc = fbgemm_amd_tbe_inplace_update(
      plan, dev_weights.numel() ? dev_weights.data_ptr() : nullptr, uvm_weights.numel() ? uvm_weights.data_ptr() : nullptr,
      update_weights.data_ptr(), update_weights.numel(), update_table_idx.data_ptr<int32_t>(), update_row_idx.data_ptr(),
      update_row_idx.scalar_type() == at::kLong ? 64 : 32, update_offsets.data_ptr<int64_t>(), n, st.data_ptr(),
      current_stream(dev_weights));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
}

// bounds_check_indices (fbgemm_gpu/codegen/utils/embedding_bounds_check_host_cpu.cpp:76-219):
// in place on indices / offsets / warning. WARNING and IGNORE repair on the
// device without a synchronization. FATAL raises where the reference's CPU
// operator raises, which costs a synchronization (the reference's GPU kernel
// asserts on the device instead).
void bounds_check_indices_hip(
    Tensor& rows_per_table, Tensor& indices, Tensor& offsets, int64_t bounds_check_mode, Tensor& warning,
    const std::optional<Tensor>& weights, const std::optional<Tensor>& B_offsets, int64_t max_B,
    const std::optional<Tensor>& /*b_t_map*/, int64_t /*info_B_num_bits*/, int64_t /*info_B_mask*/,
    int64_t /*bounds_check_version*/, bool /*prefetch_pipeline*/) {
  TORCH_CHECK(rows_per_table.is_cuda() && indices.is_cuda() && offsets.is_cuda() && warning.is_cuda(),
              "fbgemm_amd: tensors must be on the GPU");
  TORCH_CHECK(indices.scalar_type() == at::kInt || indices.scalar_type() == at::kLong, "indices must be int32 or int64");
  TORCH_CHECK(offsets.scalar_type() == indices.scalar_type(), "indices and offsets must have the same dtype");
  TORCH_CHECK(indices.is_contiguous() && offsets.is_contiguous(), "indices and offsets are modified in place and must be contiguous");
  TORCH_CHECK(warning.scalar_type() == at::kLong && warning.numel() >= 1);
  if (weights && weights->numel() != 0)
    TORCH_CHECK(weights->size(0) == indices.numel(), "weights size ", weights->size(0), " is not equal to indices size ", indices.numel());
  if (B_offsets) TORCH_CHECK(max_B >= 0);
  const Tensor rpt = rows_per_table.to(at::kLong).contiguous();
  Tensor bo;
  if (B_offsets) bo = B_offsets->to(at::kInt).contiguous();
  Tensor st;
  if (bounds_check_mode == 0) {
    st = at::zeros({4}, indices.options().dtype(at::kInt));
    TORCH_CHECK(fbgemm_amd_status_clear(st.data_ptr(), current_stream(indices)) == 0, fbgemm_amd_last_error());
  }
  const int rc = fbgemm_amd_bounds_check_indices(
      rpt.data_ptr<int64_t>(), (int32_t)rpt.numel(), indices.data_ptr(), offsets.data_ptr(),
      indices.scalar_type() == at::kLong ? 64 : 32, indices.numel(), offsets.numel(), (int32_t)bounds_check_mode,
      warning.data_ptr<int64_t>(), bo.defined() ? bo.data_ptr<int32_t>() : nullptr, st.defined() ? st.data_ptr() : nullptr,
      current_stream(indices));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  if (bounds_check_mode == 0) {
    int32_t bits = 0;
    int64_t pos = -1;
    TORCH_CHECK(fbgemm_amd_status_read(st.data_ptr(), current_stream(indices), &bits, &pos) == 0, fbgemm_amd_last_error());
    TORCH_CHECK(!(bits & FBGEMM_AMD_ERR_LENGTH_MISMATCH), "bounds_check_indices: the last offset is not the number of indices");
    TORCH_CHECK(!(bits & FBGEMM_AMD_ERR_BAG_OVERRUN), "bounds_check_indices: offsets are negative, decreasing or beyond the number of indices");
    TORCH_CHECK(!(bits & FBGEMM_AMD_ERR_INDEX_OUT_OF_RANGE), "bounds_check_indices: index at position ", pos, " is out of bounds");
  }
}

Tensor pruned_hashmap_lookup_hip(Tensor indices, Tensor offsets, Tensor hash_table, Tensor hash_table_offsets) {
  TORCH_CHECK(indices.is_cuda() && offsets.is_cuda() && hash_table.is_cuda() && hash_table_offsets.is_cuda());
  TORCH_CHECK(indices.scalar_type() == offsets.scalar_type(), "indices and offsets must have the same dtype");
  indices = indices.contiguous();
  offsets = offsets.contiguous();
  hash_table = hash_table.contiguous();
  const Tensor hto = hash_table_offsets.to(at::kLong).contiguous();
  const int64_t T = hto.numel() - 1;
  TORCH_CHECK(T > 0 && (offsets.numel() - 1) / T > 0); // embedding_forward_quantized_cpu_template.cpp:537
  Tensor dense = at::empty_like(indices);
  const int rc = fbgemm_amd_pruned_hashmap_lookup(
      indices.data_ptr(), offsets.data_ptr(), indices.scalar_type() == at::kLong ? 64 : 32, offsets.numel(),
      hash_table.data_ptr(), hash_table.scalar_type() == at::kLong ? 64 : 32, hto.data_ptr<int64_t>(), (int32_t)T,
      dense.data_ptr(), current_stream(indices));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  return dense;
}

// Row-wise quantizers (fbgemm_gpu/src/quantize_ops/quantize_ops_cpu.cpp:44-330):
// shapes and checks as the CPU operators have them.
Tensor quantize_rows(const Tensor& input, int64_t bit_rate, bool sb_float) {
  TORCH_CHECK(input.is_cuda(), "fbgemm_amd: tensors must be on the GPU");
  TORCH_CHECK(input.dim() >= 2, "Tensor 'input' must have >= 2 dimension(s). Found ", input.dim());
  TORCH_CHECK(input.scalar_type() == at::kFloat || input.scalar_type() == at::kHalf, "input must be float or half");
  const Tensor in = input.contiguous();
  const int64_t ncols = in.size(-1);
  const int64_t nrows = ncols ? in.numel() / ncols : 0;
  const int64_t epb = 8 / bit_rate;
  const int64_t out_cols = (ncols + epb - 1) / epb + (sb_float ? 8 : 4);
  auto dims = in.sizes().vec();
  dims.back() = out_cols;
  Tensor out = at::empty(dims, in.options().dtype(at::kByte));
  if (nrows == 0 || ncols == 0) return out;
  const int rc = fbgemm_amd_quantize_rowwise(
      in.data_ptr(), in.scalar_type() == at::kHalf ? FBGEMM_AMD_FP16 : FBGEMM_AMD_FP32, nrows, (int32_t)ncols,
      (int32_t)bit_rate, sb_float ? 1 : 0, FBGEMM_AMD_QLAYOUT_TRAILER, out_cols, out.data_ptr(), current_stream(in));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  return out;
}

Tensor dequantize_rows(const Tensor& input, int64_t bit_rate, bool sb_float, bool scale_bias_last, int64_t output_dtype) {
  TORCH_CHECK(input.is_cuda(), "fbgemm_amd: tensors must be on the GPU");
  TORCH_CHECK(input.dim() >= 2, "Tensor 'input' must have >= 2 dimension(s). Found ", input.dim());
  TORCH_CHECK(input.scalar_type() == at::kByte, "input must be uint8");
  const Tensor in = input.contiguous();
  const int64_t in_cols = in.size(-1);
  const int64_t nrows = in_cols ? in.numel() / in_cols : 0;
  // the column count follows from the bytes of a row (src/QuantUtils.cc:758-760, :855-856)
  const int64_t cols = (in_cols - (sb_float ? 8 : 4)) * (8 / bit_rate);
  TORCH_CHECK(cols >= 0, "rows are shorter than their scale and bias");
  auto dims = in.sizes().vec();
  dims.back() = cols;
  Tensor out = at::empty(dims, in.options().dtype(out_scalar_type(output_dtype)));
  if (nrows == 0 || cols == 0) return out;
  const int rc = fbgemm_amd_dequantize_rowwise(
      in.data_ptr(), nrows, in_cols, (int32_t)cols, (int32_t)bit_rate, sb_float ? 1 : 0,
      scale_bias_last ? FBGEMM_AMD_QLAYOUT_TRAILER : FBGEMM_AMD_QLAYOUT_TBE, (int32_t)output_dtype, out.data_ptr(),
      current_stream(in));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  return out;
}

Tensor float_to_fused8bit(const Tensor& t) { return quantize_rows(t, 8, true); }
Tensor fused8bit_to_float(const Tensor& t) { return dequantize_rows(t, 8, true, true, FBGEMM_AMD_FP32); }
Tensor fused8bit_to_half(const Tensor& t) { return dequantize_rows(t, 8, true, true, FBGEMM_AMD_FP16); }
Tensor fused8bit_to_bfloat16(const Tensor& t) { return dequantize_rows(t, 8, true, true, FBGEMM_AMD_BF16); }
Tensor fused8bit_to_float_or_half(const Tensor& t, int64_t output_dtype, bool scale_bias_last, bool quant_padding_float_type) {
  TORCH_CHECK(quant_padding_float_type || !scale_bias_last,
              "2-byte padding (quant_padding_float_type=false) only works with scale_bias_last=false");
  TORCH_CHECK(quant_padding_float_type == scale_bias_last,
              "fbgemm_amd: rows are (data, fp32 scale, fp32 bias) or (fp16 scale, fp16 bias, data)");
  return dequantize_rows(t, 8, quant_padding_float_type, scale_bias_last, output_dtype);
}
Tensor float_to_fusednbit(const Tensor& t, int64_t bit_rate) {
  TORCH_CHECK(t.dim() == 2, "Tensor 'input' must have 2 dimension(s). Found ", t.dim());
  TORCH_CHECK(bit_rate == 2 || bit_rate == 4 || bit_rate == 8, "bit_rate must be 2, 4 or 8");
  TORCH_CHECK(t.size(1) % (2 * (8 / bit_rate)) == 0,
              "ncols needs to be multiple of 2 Bytes (half type size) to make the address aligned");
  return quantize_rows(t, bit_rate, false);
}
Tensor fusednbit_to_float(const Tensor& t, int64_t bit_rate) { return dequantize_rows(t, bit_rate, false, true, FBGEMM_AMD_FP32); }
Tensor fusednbit_to_half(const Tensor& t, int64_t bit_rate) { return dequantize_rows(t, bit_rate, false, true, FBGEMM_AMD_FP16); }
Tensor fusednbit_to_float_or_half(const Tensor& t, int64_t bit_rate, int64_t output_dtype, bool scale_bias_last) {
  return dequantize_rows(t, bit_rate, false, scale_bias_last, output_dtype);
}
Tensor fusednbit_sbfront_to_float_or_half(const Tensor& t, int64_t bit_rate, int64_t output_dtype) {
  return dequantize_rows(t, bit_rate, false, false, output_dtype);
}

// FloatToHFP8Quantized / HFP8QuantizedToFloat (fbgemm_gpu/src/quantize_ops/quantize_ops_cpu.cpp:571-620)
Tensor float_to_hfp8(const Tensor& input, int64_t ebits, int64_t exponent_bias, double max_pos) {
  TORCH_CHECK(input.is_cuda(), "fbgemm_amd: tensors must be on the GPU");
  TORCH_CHECK(input.dim() == 2, "Tensor 'input' must have 2 dimension(s). Found ", input.dim());
  TORCH_CHECK(input.scalar_type() == at::kFloat, "input must be float32");
  const Tensor in = input.contiguous();
  Tensor out = at::empty(in.sizes(), in.options().dtype(at::kByte));
  const int rc = fbgemm_amd_float_to_hfp8(in.data_ptr<float>(), in.numel(), (int32_t)ebits, (int32_t)exponent_bias,
                                          (float)max_pos, out.data_ptr<uint8_t>(), current_stream(in));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  return out;
}
Tensor hfp8_to_float(const Tensor& input, int64_t ebits, int64_t exponent_bias) {
  TORCH_CHECK(input.is_cuda(), "fbgemm_amd: tensors must be on the GPU");
  TORCH_CHECK(input.dim() == 2, "Tensor 'input' must have 2 dimension(s). Found ", input.dim());
  TORCH_CHECK(input.scalar_type() == at::kByte, "input must be uint8");
  const Tensor in = input.contiguous();
  Tensor out = at::empty(in.sizes(), in.options().dtype(at::kFloat));
  const int rc = fbgemm_amd_hfp8_to_float(in.data_ptr<uint8_t>(), in.numel(), (int32_t)ebits, (int32_t)exponent_bias,
                                          out.data_ptr<float>(), current_stream(in));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  return out;
}

// Shape functions for tracing (DispatchKey::Meta), after the reference's
// fbgemm_gpu/fbgemm_gpu/sparse_ops.py:503-581: the output of a pooled lookup is
// [B, total_D], of a lookup without pooling [number of indices, D]; the copied-row
// outputs of the latter have the shapes this library writes.
Tensor lookup_meta(
    Tensor dev_weights, Tensor /*uvm_weights*/, Tensor /*weights_placements*/, Tensor /*weights_offsets*/,
    Tensor /*weights_tys*/, Tensor D_offsets, c10::SymInt total_D_, int64_t max_int2_D, int64_t max_int4_D,
    int64_t max_int8_D, int64_t max_float16_D, int64_t max_float32_D, Tensor indices, Tensor offsets, int64_t pooling_mode,
    std::optional<Tensor> /*indice_weights*/, int64_t output_dtype, std::optional<Tensor> /*lxu_cache_weights*/,
    std::optional<Tensor> /*lxu_cache_locations*/, std::optional<int64_t> /*row_alignment*/,
    std::optional<int64_t> max_float8_D, std::optional<int64_t> /*fp8_exponent_bits*/,
    std::optional<int64_t> /*fp8_exponent_bias*/) {
  if (pooling_mode == FBGEMM_AMD_POOL_NONE) {
    const int64_t D = std::max({max_int2_D, max_int4_D, max_int8_D, max_float16_D, max_float32_D, max_float8_D.value_or(0)});
    TORCH_CHECK(D > 0);
    if (output_dtype == FBGEMM_AMD_INT8 || output_dtype == FBGEMM_AMD_INT4)
      return at::empty({indices.numel(), output_dtype == FBGEMM_AMD_INT8 ? D + 4 : (D + 9) / 2},
                       dev_weights.options().dtype(at::kByte));
    return at::empty({indices.numel(), D}, dev_weights.options().dtype(out_scalar_type(output_dtype)));
  }
  const int64_t T = D_offsets.numel() - 1;
  const int64_t total_D = total_D_.expect_int();
  TORCH_CHECK(T > 0 && total_D > 0);
  if (output_dtype == FBGEMM_AMD_INT8)
    return at::empty({(offsets.size(0) - 1) / T, total_D + 8 * T}, dev_weights.options().dtype(at::kByte));
  return at::empty({(offsets.size(0) - 1) / T, total_D}, dev_weights.options().dtype(out_scalar_type(output_dtype)));
}
Tensor same_shape_as_indices_meta(Tensor indices, Tensor /*offsets*/, Tensor /*table*/, Tensor /*table_offsets*/) {
  return at::empty_like(indices);
}

// embedding_bag_rowwise_prune (fbgemm_gpu/src/sparse_ops/sparse_ops_cpu.cpp:2773-2893)
std::tuple<Tensor, Tensor> rowwise_prune(const Tensor& weights, const Tensor& indicator, double threshold,
                                         at::ScalarType compressed_indices_dtype, bool abs, c10::SymInt min_non_pruned_rows_,
                                         std::optional<double> min_save_ratio) {
  TORCH_CHECK(weights.is_cuda() && indicator.is_cuda(), "fbgemm_amd: tensors must be on the GPU");
  TORCH_CHECK(weights.dim() == 2, "Tensor 'weights' must have 2 dimension(s). Found ", weights.dim());
  TORCH_CHECK(indicator.numel() == weights.size(0),
              "Number of elements in 'indicator' should be equivalent to number of rows in 'weights'.");
  TORCH_CHECK(threshold >= 0.0, "Threshold should be greater than or equal to zero.");
  TORCH_CHECK(compressed_indices_dtype == at::kInt || compressed_indices_dtype == at::kLong,
              "'compressed_indices_dtype' should be Int/Long.");
  const int64_t min_rows = min_non_pruned_rows_.expect_int();
  const int64_t rows = weights.size(0), cols = weights.size(1);
  if (min_save_ratio.has_value() &&
      !((double)(rows * 4 + min_rows * cols * 4) < *min_save_ratio * (double)(4 * weights.numel()))) {
    Tensor one = at::zeros({1}, weights.options().dtype(compressed_indices_dtype));
    return {weights, one};
  }
  const Tensor w = weights.contiguous();
  const Tensor ind = indicator.to(at::kFloat).contiguous();
  Tensor remap = at::empty({rows}, w.options().dtype(compressed_indices_dtype));
  const int32_t bits = compressed_indices_dtype == at::kLong ? 64 : 32;
  int64_t kept = 0;
  int rc = fbgemm_amd_rowwise_prune_map(ind.data_ptr<float>(), rows, threshold, abs ? 1 : 0, min_rows, bits,
                                        remap.data_ptr(), &kept, current_stream(w));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  Tensor out = at::empty({kept, cols}, w.options());
  rc = fbgemm_amd_rowwise_prune_gather(w.data_ptr(), rows, cols * (int64_t)w.element_size(), remap.data_ptr(), bits,
                                       out.data_ptr(), kept, current_stream(w));
  TORCH_CHECK(rc == 0, "fbgemm_amd: ", fbgemm_amd_last_error());
  return {out, remap};
}

} // namespace

// The schema strings are the reference's, character for character. When a real
// fbgemm_gpu is loaded in the same process it has already defined them: build
// with -DFBGEMM_AMD_IMPL_ONLY to register the implementations alone.
TORCH_LIBRARY_FRAGMENT(fbgemm, m) {
#ifndef FBGEMM_AMD_IMPL_ONLY
  m.def(
      "int_nbit_split_embedding_codegen_lookup_function(Tensor dev_weights, Tensor uvm_weights, Tensor weights_placements, Tensor weights_offsets, Tensor weights_tys, Tensor D_offsets, SymInt total_D, int max_int2_D, int max_int4_D, int max_int8_D, int max_float16_D, int max_float32_D, Tensor indices, Tensor offsets, int pooling_mode, Tensor? indice_weights, int output_dtype=1, Tensor? lxu_cache_weights=None, Tensor? lxu_cache_locations=None, int? row_alignment = None, int? max_float8_D=0, int? fp8_exponent_bits=-1, int? fp8_exponent_bias=-1) -> Tensor");
  m.def(
      "pruned_array_lookup(Tensor indices, Tensor offsets, Tensor index_remappings, Tensor index_remappings_offsets) -> Tensor");
#endif
#ifndef FBGEMM_AMD_IMPL_ONLY
  m.def(
      "int_nbit_split_embedding_uvm_caching_codegen_lookup_function(Tensor dev_weights, Tensor uvm_weights, Tensor weights_placements, Tensor weights_offsets, Tensor weights_tys, Tensor D_offsets, SymInt total_D, int max_int2_D, int max_int4_D, int max_int8_D, int max_float16_D, int max_float32_D, Tensor indices, Tensor offsets, int pooling_mode, Tensor? indice_weights=None, int output_dtype=1, Tensor? lxu_cache_weights=None, Tensor? lxu_cache_locations=None, int? row_alignment=-1, int? max_float8_D=0, int? fp8_exponent_bits=-1, int? fp8_exponent_bias=-1, Tensor? cache_hash_size_cumsum=None, int? total_cache_hash_size=-1, Tensor? cache_index_table_map=None, Tensor? lxu_cache_state=None, Tensor? lxu_state=None) -> Tensor");
#endif
  m.impl("int_nbit_split_embedding_uvm_caching_codegen_lookup_function",
         torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(int_nbit_split_embedding_uvm_caching_codegen_lookup_function_hip)));
  m.impl("int_nbit_split_embedding_codegen_lookup_function",
         torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(int_nbit_split_embedding_codegen_lookup_function_hip)));
  m.impl("pruned_array_lookup", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(pruned_array_lookup_hip)));
  m.impl("int_nbit_split_embedding_codegen_lookup_function", torch::dispatch(c10::DispatchKey::Meta, TORCH_FN(lookup_meta)));
  m.impl("pruned_array_lookup", torch::dispatch(c10::DispatchKey::Meta, TORCH_FN(same_shape_as_indices_meta)));
#ifndef FBGEMM_AMD_IMPL_ONLY
  // fbgemm_gpu/src/embedding_inplace_ops/embedding_inplace_update_cpu.cpp:257-260
  m.def(
      "emb_inplace_update(Tensor(a!) dev_weights, Tensor(b!) uvm_weights, Tensor weights_placements, Tensor weights_offsets, Tensor weights_tys, Tensor D_offsets, Tensor update_weights, Tensor update_table_indices, Tensor update_row_indices, Tensor update_offsets, int row_alignment=1, Tensor(c!)? lxu_cache_weights=None, Tensor? lxu_cache_locations=None) -> ()");
  m.def(
      "pruned_array_lookup_from_row_idx(Tensor update_row_indices, Tensor update_table_indices, Tensor index_remappings, Tensor index_remappings_offsets) -> Tensor");
#endif
  m.impl("emb_inplace_update", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(emb_inplace_update_hip)));
  m.impl("pruned_array_lookup_from_row_idx", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(pruned_array_lookup_from_row_idx_hip)));
#ifndef FBGEMM_AMD_IMPL_ONLY
  // embedding_forward_quantized_host_cpu.cpp:338-341
  m.def(
      "pruned_hashmap_lookup(Tensor indices, Tensor offsets, Tensor hash_table, Tensor hash_table_offsets) -> Tensor");
  // fbgemm_gpu/codegen/utils/embedding_bounds_check_host_cpu.cpp:255-270
  m.def(
      "bounds_check_indices("
      "    Tensor rows_per_table, "
      "    Tensor(a!) indices, "
      "    Tensor(b!) offsets, "
      "    int bounds_check_mode, "
      "    Tensor(c!) warning, "
      "    Tensor(d!)? weights=None, "
      "    Tensor? B_offsets=None, "
      "    SymInt max_B=-1, "
      "    Tensor? b_t_map=None, "
      "    int info_B_num_bits=-1, "
      "    int info_B_mask=-1, "
      "    int bounds_check_version=1, "
      "    bool prefetch_pipeline=False"
      ") -> ()");
  // fbgemm_gpu/src/quantize_ops/quantize_ops_cpu.cpp:632-666
  m.def("FloatToFused8BitRowwiseQuantized(Tensor t) -> Tensor");
  m.def("HalfToFused8BitRowwiseQuantized(Tensor t) -> Tensor");
  m.def("FloatOrHalfToFused8BitRowwiseQuantized(Tensor t) -> Tensor");
  m.def("Fused8BitRowwiseQuantizedToFloat(Tensor input) -> Tensor");
  m.def("Fused8BitRowwiseQuantizedToHalf(Tensor input) -> Tensor");
  m.def("Fused8BitRowwiseQuantizedToBfloat16(Tensor input) -> Tensor");
  m.def(
      "Fused8BitRowwiseQuantizedToFloatOrHalf(Tensor input, int output_dtype=0, bool scale_bias_last=True, bool quant_padding_float_type=True) -> Tensor");
  m.def(
      "FloatToFusedNBitRowwiseQuantizedSBHalf(Tensor input, int bit_rate) -> Tensor");
  m.def(
      "HalfToFusedNBitRowwiseQuantizedSBHalf(Tensor input, int bit_rate) -> Tensor");
  m.def(
      "FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf(Tensor input, int bit_rate) -> Tensor");
  m.def(
      "FusedNBitRowwiseQuantizedSBHalfToFloat(Tensor input, int bit_rate) -> Tensor");
  m.def(
      "FusedNBitRowwiseQuantizedSBHalfFrontToFloatOrHalf(Tensor input, int bit_rate, int output_dtype) -> Tensor");
  m.def(
      "FusedNBitRowwiseQuantizedSBHalfToHalf(Tensor input, int bit_rate) -> Tensor");
  m.def(
      "FusedNBitRowwiseQuantizedSBHalfToFloatOrHalf(Tensor input, int bit_rate, int output_dtype=0, bool scale_bias_last=True) -> Tensor");
  // fbgemm_gpu/src/sparse_ops/sparse_ops_cpu.cpp:3891-3892
  m.def(
      "embedding_bag_rowwise_prune(Tensor weight, Tensor indicator, float threshold, ScalarType compressed_indices_dtype, bool abs=True, SymInt min_num_rows=0, float? min_save_ratio=1.0) -> (Tensor, Tensor)");
  // quantize_ops_cpu.cpp:670-673
  m.def("FloatToHFP8Quantized(Tensor input, int ebits, int exponent_bias, float max_pos) -> Tensor");
  m.def("HFP8QuantizedToFloat(Tensor input, int ebits, int exponent_bias) -> Tensor");
#endif
  m.impl("embedding_bag_rowwise_prune", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(rowwise_prune)));
  m.impl("FloatToHFP8Quantized", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(float_to_hfp8)));
  m.impl("HFP8QuantizedToFloat", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(hfp8_to_float)));
  m.impl("pruned_hashmap_lookup", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(pruned_hashmap_lookup_hip)));
  m.impl("pruned_hashmap_lookup", torch::dispatch(c10::DispatchKey::Meta, TORCH_FN(same_shape_as_indices_meta)));
  m.impl("bounds_check_indices", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(bounds_check_indices_hip)));
  m.impl("FloatToFused8BitRowwiseQuantized", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(float_to_fused8bit)));
  m.impl("HalfToFused8BitRowwiseQuantized", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(float_to_fused8bit)));
  m.impl("FloatOrHalfToFused8BitRowwiseQuantized", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(float_to_fused8bit)));
  m.impl("Fused8BitRowwiseQuantizedToFloat", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(fused8bit_to_float)));
  m.impl("Fused8BitRowwiseQuantizedToHalf", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(fused8bit_to_half)));
  m.impl("Fused8BitRowwiseQuantizedToBfloat16", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(fused8bit_to_bfloat16)));
  m.impl("Fused8BitRowwiseQuantizedToFloatOrHalf", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(fused8bit_to_float_or_half)));
  m.impl("FloatToFusedNBitRowwiseQuantizedSBHalf", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(float_to_fusednbit)));
  m.impl("HalfToFusedNBitRowwiseQuantizedSBHalf", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(float_to_fusednbit)));
  m.impl("FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(float_to_fusednbit)));
  m.impl("FusedNBitRowwiseQuantizedSBHalfToFloat", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(fusednbit_to_float)));
  m.impl("FusedNBitRowwiseQuantizedSBHalfToHalf", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(fusednbit_to_half)));
  m.impl("FusedNBitRowwiseQuantizedSBHalfToFloatOrHalf", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(fusednbit_to_float_or_half)));
  m.impl("FusedNBitRowwiseQuantizedSBHalfFrontToFloatOrHalf", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(fusednbit_sbfront_to_float_or_half)));
}

TORCH_LIBRARY_FRAGMENT(fbgemm_amd, m) {
  m.def("lookup_status(Tensor like) -> int");
  m.impl("lookup_status", torch::dispatch(c10::DispatchKey::CUDA, TORCH_FN(lookup_status)));
}
