// Drives the C++ factory templates of include/fbgemm_amd_embedding.hpp the way
// the reference's gtests drive fbgemm::GenerateEmbeddingSpMDM*
// (test/EmbeddingSpMDMNBitTest.cc:92-418, test/EmbeddingSpMDM8BitTest.cc:82-372):
// random table, random bags, optimized kernel vs the scalar oracle, every
// output bit equal, ten sentinel values after the output untouched, and the
// corner cases (empty indices, out-of-range index, lengths-sum mismatch)
// returning false. Exit code 0 = all cases passed.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <random>
#include <thread>
#include <vector>

#include "../../include/fbgemm_amd_embedding.hpp"

extern "C" int oracle_embedding_spmdm(
    int in_ty, int64_t block_size, int64_t output_size, int64_t index_size, int64_t data_size, const void* input,
    const void* indices, int idx64, const void* offsets_or_lengths, int off64, const float* weights,
    int normalize_by_lengths, void* out, int out_ty, int is_weight_positional, int use_offsets,
    int64_t output_stride, int64_t input_stride, int scale_bias_last, const int32_t* remap);
extern "C" uint16_t oracle_float2half_rn(float f);
extern "C" int oracle_embedding_spmdm_nobag(
    int in_ty, int64_t block_size, int64_t output_size, int64_t data_size, const void* input, const void* indices,
    int idx64, const float* weights, void* out, int out_ty, int64_t output_stride, int64_t input_stride,
    int scale_bias_last);
extern "C" int oracle_embedding_spmdm_fp8(
    int64_t block_size, int64_t output_size, int64_t index_size, int64_t data_size, const uint8_t* input,
    const void* indices, int idx64, const void* offsets_or_lengths, int off64, const float* weights,
    int normalize_by_lengths, void* out, int out_ty, int is_weight_positional, int use_offsets,
    int64_t output_stride, int64_t input_stride, int exponent_bits, int exponent_bias, int skip_minus_one);
extern "C" void oracle_quantize_rowwise(const void* input, int half_in, int64_t rows, int32_t cols, int32_t bit_rate,
                                        int32_t sb_float, int32_t layout, int64_t out_stride, uint8_t* output);
extern "C" void oracle_quantize_rowwise_min_max(const void* input, int half_in, int64_t rows, int32_t cols,
                                                int32_t bit_rate, int32_t sb_float, int32_t layout, int64_t out_stride,
                                                uint8_t* output, const void* min_max);
extern "C" void oracle_dequantize_rowwise(const uint8_t* input, int64_t rows, int64_t in_stride, int32_t cols,
                                          int32_t bit_rate, int32_t sb_float, int32_t layout, int32_t output_ty,
                                          void* output);

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e_)); return 2; } } while (0)

template <typename T>
struct Dev {
  T* p = nullptr;
  size_t n = 0;
  explicit Dev(const std::vector<T>& h) : n(h.size()) {
    (void)hipMalloc((void**)&p, std::max<size_t>(n, 1) * sizeof(T));
    if (n) (void)hipMemcpy(p, h.data(), n * sizeof(T), hipMemcpyHostToDevice);
  }
  ~Dev() { (void)hipFree(p); }
  std::vector<T> host() const {
    std::vector<T> h(n);
    if (n) (void)hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost);
    return h;
  }
};

static std::atomic<int> failures{0};
#define CHECK(cond, ...) do { if (!(cond)) { ++failures; printf("FAIL %s:%d: ", __FILE__, __LINE__); printf(__VA_ARGS__); printf("\n"); } } while (0)

template <typename IndexType, typename OffsetType, typename OutType>
void run_nbit(int bit_rate, int64_t D, int batch, int rows, int avg_len, bool weighted, bool normalize, bool use_offsets,
              int corner /*0 none, 1 empty indices, 2 out-of-range, 3 unmatched lengths*/, unsigned seed) {
  std::mt19937 rng(seed);
  const int epb = 8 / bit_rate;
  const int64_t stride = (D + epb - 1) / epb + 4;
  std::vector<uint8_t> table(rows * stride);
  for (auto& b : table) b = rng() & 0xff;
  for (int r = 0; r < rows; ++r) {
    uint16_t sb[2] = {oracle_float2half_rn(0.01f + 0.09f * (rng() % 1000) / 1000.f),
                      oracle_float2half_rn(-1.f + 2.f * (rng() % 1000) / 1000.f)};
    memcpy(&table[r * stride + stride - 4], sb, 4);
  }
  std::vector<OffsetType> lengths(batch), offsets(batch + 1, 0);
  for (int b = 0; b < batch; ++b) {
    lengths[b] = corner == 1 ? 0 : 1 + rng() % (2 * avg_len);
    offsets[b + 1] = offsets[b] + lengths[b];
  }
  int64_t n = offsets[batch];
  std::vector<IndexType> indices(n);
  for (auto& i : indices) i = rng() % rows;
  if (n) indices[0] = rows - 1;
  if (corner == 2 && n) indices[n / 2] = rows;
  int64_t index_size = n;
  if (corner == 3) { index_size = n + 1; indices.push_back(0); }
  std::vector<float> w(indices.size());
  for (auto& x : w) x = (float)(rng() % 2000) / 1000.f - 1.f;

  const int out_ty = std::is_same_v<OutType, float> ? FBGEMM_AMD_FP32 : FBGEMM_AMD_FP16;
  constexpr int kSentinels = 10;
  std::vector<OutType> out_ref(batch * D + kSentinels), out_init(batch * D + kSentinels);
  OutType sentinel;
  memset(&sentinel, 0xAB, sizeof(sentinel));
  for (auto& o : out_init) o = sentinel;
  out_ref = out_init;
  const int ok_ref = oracle_embedding_spmdm(
      bit_rate == 4 ? FBGEMM_AMD_INT4 : FBGEMM_AMD_INT2, D, batch, index_size, rows, table.data(), indices.data(),
      sizeof(IndexType) == 8, use_offsets ? (const void*)offsets.data() : (const void*)lengths.data(),
      sizeof(OffsetType) == 8, weighted ? w.data() : nullptr, normalize, out_ref.data(), out_ty, 0, use_offsets, -1, -1, 1,
      nullptr);

  Dev<uint8_t> d_table(table);
  Dev<IndexType> d_idx(indices);
  Dev<OffsetType> d_off(use_offsets ? offsets : lengths);
  Dev<float> d_w(w);
  Dev<OutType> d_out(out_init);
  auto kernel = fbgemm_amd::GenerateEmbeddingSpMDMNBit<IndexType, OffsetType, OutType>(
      bit_rate, D, weighted, normalize, 16, false, use_offsets);
  const bool ok = kernel(batch, index_size, rows, d_table.p, d_idx.p, d_off.p, weighted ? d_w.p : nullptr, d_out.p);
  CHECK(ok == (ok_ref != 0), "return value %d vs oracle %d (bit_rate %d D %ld corner %d)", (int)ok, ok_ref, bit_rate, (long)D, corner);
  if (ok && ok_ref) {
    auto got = d_out.host();
    CHECK(memcmp(got.data(), out_ref.data(), got.size() * sizeof(OutType)) == 0,
          "output differs (bit_rate %d D %ld batch %d weighted %d normalize %d use_offsets %d)", bit_rate, (long)D, batch,
          weighted, normalize, use_offsets);
  }
}

template <typename IndexType, typename OffsetType>
void run_8bit(int64_t D, int batch, int rows, int avg_len, bool weighted, bool normalize, unsigned seed) {
  std::mt19937 rng(seed);
  const int64_t stride = D + 8;
  std::vector<uint8_t> table(rows * stride);
  for (auto& b : table) b = rng() & 0xff;
  for (int r = 0; r < rows; ++r) {
    float sb[2] = {0.001f + 0.009f * (rng() % 1000) / 1000.f, -1.f + 2.f * (rng() % 1000) / 1000.f};
    memcpy(&table[r * stride + D], sb, 8);
  }
  std::vector<OffsetType> offsets(batch + 1, 0);
  for (int b = 0; b < batch; ++b) offsets[b + 1] = offsets[b] + 1 + rng() % (2 * avg_len);
  std::vector<IndexType> indices(offsets[batch]);
  for (auto& i : indices) i = rng() % rows;
  std::vector<float> w(indices.size());
  for (auto& x : w) x = (float)(rng() % 2000) / 1000.f - 1.f;
  std::vector<float> out_ref(batch * D, 0.f), out_init(batch * D, -7.f);
  const int ok_ref = oracle_embedding_spmdm(FBGEMM_AMD_INT8, D, batch, indices.size(), rows, table.data(), indices.data(),
                                            sizeof(IndexType) == 8, offsets.data(), sizeof(OffsetType) == 8,
                                            weighted ? w.data() : nullptr, normalize, out_ref.data(), FBGEMM_AMD_FP32, 0, 1,
                                            -1, -1, 1, nullptr);
  Dev<uint8_t> d_table(table);
  Dev<IndexType> d_idx(indices);
  Dev<OffsetType> d_off(offsets);
  Dev<float> d_w(w);
  Dev<float> d_out(out_init);
  auto kernel = fbgemm_amd::GenerateEmbeddingSpMDM<uint8_t, IndexType, OffsetType, float>(D, weighted, normalize);
  const bool ok = kernel(batch, indices.size(), rows, d_table.p, d_idx.p, d_off.p, weighted ? d_w.p : nullptr, d_out.p);
  CHECK(ok && ok_ref, "8-bit lookup rejected valid input");
  auto got = d_out.host();
  CHECK(memcmp(got.data(), out_ref.data(), got.size() * 4) == 0, "8-bit output differs (D %ld weighted %d normalize %d)",
        (long)D, weighted, normalize);
}

// no_bag of the 8-bit factory (float rows out, and rows copied as stored) and of the 4-bit one,
// and the 8-bit-float factory, against the oracle.
template <typename IndexType>
void run_no_bag_and_fp8(int64_t D, int n, int rows, unsigned seed) {
  std::mt19937 rng(seed);
  const int64_t stride = D + 8;
  std::vector<uint8_t> table(rows * stride);
  for (auto& b : table) b = rng() & 0xff;
  for (int r = 0; r < rows; ++r) {
    float sb[2] = {0.001f + 0.009f * (rng() % 1000) / 1000.f, -1.f + 2.f * (rng() % 1000) / 1000.f};
    memcpy(&table[r * stride + D], sb, 8);
  }
  std::vector<IndexType> indices(n);
  for (auto& i : indices) i = rng() % rows;
  std::vector<float> w(n);
  for (auto& x : w) x = (float)(rng() % 2000) / 1000.f - 1.f;
  Dev<uint8_t> d_table(table);
  Dev<IndexType> d_idx(indices);
  Dev<float> d_w(w);
  const int idx64 = sizeof(IndexType) == 8;
  {
    std::vector<float> want(n * D, -7.f), init(n * D, -7.f);
    const int ok_ref = oracle_embedding_spmdm_nobag(FBGEMM_AMD_INT8, D, n, rows, table.data(), indices.data(), idx64, w.data(),
                                                    want.data(), FBGEMM_AMD_FP32, -1, -1, 1);
    Dev<float> d_out(init);
    auto kernel = fbgemm_amd::GenerateEmbeddingSpMDMWithStrides<uint8_t, IndexType, int32_t, float>(
        D, true, false, 16, false, true, -1, -1, true, /*no_bag=*/true);
    const bool ok = kernel(n, n, rows, d_table.p, d_idx.p, nullptr, d_w.p, d_out.p);
    auto got = d_out.host();
    CHECK(ok && ok_ref && memcmp(got.data(), want.data(), got.size() * 4) == 0, "no_bag 8-bit -> float differs (D %ld)", (long)D);
  }
  {
    std::vector<uint8_t> want(n * stride, 0xA5), init(n * stride, 0xA5);
    const int ok_ref = oracle_embedding_spmdm_nobag(FBGEMM_AMD_INT8, D, n, rows, table.data(), indices.data(), idx64, nullptr,
                                                    want.data(), FBGEMM_AMD_INT8, stride, -1, 1);
    Dev<uint8_t> d_out(init);
    auto kernel = fbgemm_amd::GenerateEmbeddingSpMDMWithStrides<uint8_t, IndexType, int32_t, uint8_t>(
        D, false, false, 16, false, true, stride, -1, true, /*no_bag=*/true);
    const bool ok = kernel(n, n, rows, d_table.p, d_idx.p, nullptr, nullptr, d_out.p);
    auto got = d_out.host();
    CHECK(ok && ok_ref && got == want, "no_bag 8-bit row copy differs (D %ld)", (long)D);
  }
  if (D % 2 == 0) {
    const int64_t s4 = D / 2 + 4;
    std::vector<uint8_t> t4(rows * s4);
    for (auto& b : t4) b = rng() & 0xff;
    std::vector<uint8_t> want(n * s4, 0xA5), init(n * s4, 0xA5);
    const int ok_ref = oracle_embedding_spmdm_nobag(FBGEMM_AMD_INT4, D, n, rows, t4.data(), indices.data(), idx64, nullptr,
                                                    want.data(), FBGEMM_AMD_INT4, -1, -1, 0);
    Dev<uint8_t> d_t4(t4), d_out(init);
    auto kernel = fbgemm_amd::GenerateEmbeddingSpMDMNBitWithStrides<IndexType, int32_t, uint8_t>(
        4, D, false, false, 16, false, true, -1, -1, false, false, /*no_bag=*/true, /*output_bit_rate=*/4);
    const bool ok = kernel(n, n, rows, d_t4.p, d_idx.p, nullptr, nullptr, d_out.p);
    auto got = d_out.host();
    CHECK(ok && ok_ref && got == want, "no_bag 4-bit row copy differs (D %ld)", (long)D);
    auto none = fbgemm_amd::GenerateEmbeddingSpMDMNBitWithStrides<IndexType, int32_t, float>(
        4, D, false, false, 16, false, true, -1, -1, false, false, /*no_bag=*/true);
    CHECK(!none(n, n, rows, d_t4.p, d_idx.p, nullptr, nullptr, nullptr), "no_bag 4-bit -> float must return false");
  }
  {
    // pooled 8-bit floats: bags of up to 7, weighted, mean
    std::vector<int32_t> offsets(1, 0);
    while (offsets.back() < n) offsets.push_back(std::min<int32_t>(n, offsets.back() + rng() % 8));
    const int batch = (int)offsets.size() - 1;
    std::vector<uint8_t> t8(rows * D);
    for (auto& b : t8) b = rng() & 0xff;
    std::vector<uint16_t> want(batch * D, 0), init(batch * D, 0xBEEF);
    const int ok_ref = oracle_embedding_spmdm_fp8(D, batch, n, rows, t8.data(), indices.data(), idx64, offsets.data(), 0,
                                                  w.data(), 1, want.data(), FBGEMM_AMD_FP16, 0, 1, -1, -1, 4, 7, 0);
    Dev<uint8_t> d_t8(t8);
    Dev<int32_t> d_off(offsets);
    Dev<uint16_t> d_out(init);
    auto kernel = fbgemm_amd::GenerateEmbeddingSpMDMFP8WithStrides<IndexType, int32_t, uint16_t>(D, true);
    const bool ok = kernel(batch, n, rows, d_t8.p, d_idx.p, d_off.p, d_w.p, d_out.p);
    auto got = d_out.host();
    CHECK(ok && ok_ref && got == want, "8-bit-float pooled lookup differs (D %ld)", (long)D);
  }
}

extern "C" void oracle_compressed_indices_remap(
    int32_t offsets_len, const void* indices, int idx64, const int32_t* mapping, const void* offsets, const float* weights,
    void* out_indices, void* out_offsets, float* out_weights);

// compressed_indices_remap against the oracle (after test/EmbeddingSpMDMTest.cc:1040-1192: half of the rows pruned)
template <typename IndexType>
void run_remap(int batch, int rows, int avg_len, bool weighted, unsigned seed) {
  std::mt19937 rng(seed);
  std::vector<int32_t> mapping(rows);
  int32_t next = 0;
  for (auto& m : mapping) m = (rng() & 1) ? next++ : -1;
  std::vector<IndexType> offsets(batch + 1, 0);
  for (int b = 0; b < batch; ++b) offsets[b + 1] = offsets[b] + rng() % (2 * avg_len + 1);
  std::vector<IndexType> indices(offsets[batch]);
  for (auto& i : indices) i = rng() % rows;
  std::vector<float> w(indices.size());
  for (auto& x : w) x = (float)(rng() % 2000) / 1000.f - 1.f;
  std::vector<IndexType> want_i(indices.size(), 0), want_o(offsets.size(), 0);
  std::vector<float> want_w(w.size(), 0.f);
  oracle_compressed_indices_remap((int32_t)offsets.size(), indices.data(), sizeof(IndexType) == 8, mapping.data(),
                                  offsets.data(), weighted ? w.data() : nullptr, want_i.data(), want_o.data(), want_w.data());
  Dev<IndexType> d_idx(indices), d_off(offsets), d_oi(want_i), d_oo(want_o);
  Dev<int32_t> d_map(mapping);
  Dev<float> d_w(w), d_ow(want_w);
  fbgemm_amd::compressed_indices_remap<IndexType>((int32_t)offsets.size(), d_idx.p, d_map.p, d_off.p, weighted ? d_w.p : nullptr,
                                                  d_oi.p, d_oo.p, weighted ? d_ow.p : nullptr);
  const auto got_i = d_oi.host();
  const auto got_o = d_oo.host();
  const auto got_w = d_ow.host();
  const size_t n = (size_t)want_o.back();
  CHECK(got_o == want_o, "remap offsets differ (batch %d)", batch);
  CHECK(std::equal(got_i.begin(), got_i.begin() + n, want_i.begin()), "remap indices differ (batch %d)", batch);
  if (weighted) CHECK(memcmp(got_w.data(), want_w.data(), n * 4) == 0, "remap weights differ (batch %d)", batch);
}

// The quantizer templates (names and arguments of include/fbgemm/QuantUtils.h:276-334)
// against the oracle, after test/QuantUtilsTest.cc's fused row-wise cases.
void run_quantizers(int rows, int cols, unsigned seed) {
  std::mt19937 rng(seed);
  std::vector<float> x((size_t)rows * cols);
  for (auto& v : x) v = (float)((int)(rng() % 20001) - 10000) / 1000.f;
  Dev<float> d_x(x);
  for (int bit_rate : {2, 4, 8}) {
    const int epb = 8 / bit_rate;
    if (cols % epb) continue;
    const int stride = cols / epb + 4;
    std::vector<uint8_t> want((size_t)rows * stride), zero((size_t)rows * stride, 0);
    oracle_quantize_rowwise(x.data(), 0, rows, cols, bit_rate, 0, 0, stride, want.data());
    Dev<uint8_t> d_q(zero);
    fbgemm_amd::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf<float>(bit_rate, d_x.p, rows, cols, d_q.p);
    CHECK(d_q.host() == want, "%d-bit rows differ (%d x %d)", bit_rate, rows, cols);
    std::vector<float> back_want((size_t)rows * cols), back_init((size_t)rows * cols, -3.f);
    oracle_dequantize_rowwise(want.data(), rows, stride, cols, bit_rate, 0, 0, FBGEMM_AMD_FP32, back_want.data());
    Dev<float> d_back(back_init);
    fbgemm_amd::FusedNBitRowwiseQuantizedSBHalfToFloatOrHalf<float>(bit_rate, d_q.p, rows, stride, d_back.p);
    auto got = d_back.host();
    CHECK(memcmp(got.data(), back_want.data(), got.size() * 4) == 0, "%d-bit rows dequantize differently", bit_rate);
  }
  const int stride8 = cols + 8;
  std::vector<uint8_t> want8((size_t)rows * stride8), zero8((size_t)rows * stride8, 0);
  oracle_quantize_rowwise(x.data(), 0, rows, cols, 8, 1, 0, stride8, want8.data());
  Dev<uint8_t> d_q8(zero8);
  fbgemm_amd::FloatOrHalfToFused8BitRowwiseQuantizedSBFloat<float>(d_x.p, rows, cols, d_q8.p);
  CHECK(d_q8.host() == want8, "8-bit rows with fp32 scale/bias differ (%d x %d)", rows, cols);
  std::vector<uint16_t> half_want((size_t)rows * cols), half_init((size_t)rows * cols, 0xBEEF);
  oracle_dequantize_rowwise(want8.data(), rows, stride8, cols, 8, 1, 0, FBGEMM_AMD_FP16, half_want.data());
  Dev<uint16_t> d_half(half_init);
  fbgemm_amd::Fused8BitRowwiseQuantizedSBFloatToFloatOrHalf<std::uint16_t>(d_q8.p, rows, stride8, d_half.p);
  CHECK(d_half.host() == half_want, "8-bit rows dequantize to fp16 differently");

  // extremes from the caller, narrower than the rows' own, so that the clamping rules show
  std::vector<float> mm((size_t)rows * 2);
  for (int r = 0; r < rows; ++r) {
    mm[2 * r] = -4.f + (float)(rng() % 1000) / 500.f;
    mm[2 * r + 1] = 2.f + (float)(rng() % 1000) / 500.f;
  }
  Dev<float> d_mm(mm);
  for (int bit_rate : {2, 4, 8}) {
    const int epb = 8 / bit_rate;
    if (cols % epb) continue;
    const int stride = cols / epb + 4;
    std::vector<uint8_t> want((size_t)rows * stride), zero((size_t)rows * stride, 0);
    oracle_quantize_rowwise_min_max(x.data(), 0, rows, cols, bit_rate, 0, 0, stride, want.data(), mm.data());
    Dev<uint8_t> d_q(zero);
    fbgemm_amd::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf<float>(bit_rate, d_x.p, rows, cols, d_q.p, d_mm.p);
    CHECK(d_q.host() == want, "%d-bit rows with the caller's extremes differ (%d x %d)", bit_rate, rows, cols);
  }
  oracle_quantize_rowwise_min_max(x.data(), 0, rows, cols, 8, 1, 0, stride8, want8.data(), mm.data());
  Dev<uint8_t> d_q8m(zero8);
  fbgemm_amd::FloatOrHalfToFused8BitRowwiseQuantizedSBFloat<float>(d_x.p, rows, cols, d_q8m.p, d_mm.p);
  CHECK(d_q8m.host() == want8, "8-bit rows with the caller's extremes differ (%d x %d)", rows, cols);
}

// The reference's fixed-number case (test/QuantUtilsTest.cc:547-611, :851-945): two rows of four,
// their extremes handed in, and the bytes its authors worked out by hand.
void run_fixed_numbers() {
  const std::vector<float> x = {1, 1, 1, 1, -64, -2.75f, 61.625f, 191};
  const std::vector<float> mm = {1, 1, -64, 191};
  Dev<float> d_x(x), d_mm(mm);
  const std::vector<uint8_t> want8h = {0, 0, 0, 0, 0x00, 0x3c, 0x00, 0x3c, 0, 61, 126, 255, 0x00, 0x3c, 0x00, 0xd4};
  const std::vector<uint8_t> want4 = {0x00, 0x00, 0x00, 0x3c, 0x00, 0x3c, 0x40, 0xf7, 0x40, 0x4c, 0x00, 0xd4};
  const std::vector<uint8_t> want2 = {0x00, 0x00, 0x3c, 0x00, 0x3c, 0xd4, 0x50, 0x55, 0x00, 0xd4};
  const std::vector<uint8_t> want8f = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0x80, 0x3f, 0, 61, 126, 255, 0, 0, 0x80, 0x3f, 0, 0, 0x80, 0xc2};
  for (int with = 0; with < 2; ++with) {
    const float* extremes = with ? d_mm.p : nullptr;
    for (int bit_rate : {2, 4, 8}) {
      const auto& want = bit_rate == 2 ? want2 : bit_rate == 4 ? want4 : want8h;
      Dev<uint8_t> d_q(std::vector<uint8_t>(want.size(), 0));
      fbgemm_amd::FloatOrHalfToFusedNBitRowwiseQuantizedSBHalf<float>(bit_rate, d_x.p, 2, 4, d_q.p, extremes);
      CHECK(d_q.host() == want, "fixed numbers, %d bits, extremes %s", bit_rate, with ? "given" : "found");
    }
    Dev<uint8_t> d_q(std::vector<uint8_t>(want8f.size(), 0));
    fbgemm_amd::FloatOrHalfToFused8BitRowwiseQuantizedSBFloat<float>(d_x.p, 2, 4, d_q.p, extremes);
    CHECK(d_q.host() == want8f, "fixed numbers, 8 bits with fp32 pair, extremes %s", with ? "given" : "found");
  }
}

int main() {
  int ndev = 0;
  HIP_OK(hipGetDeviceCount(&ndev));
  if (ndev == 0) { printf("no GPU\n"); return 3; }
  // shapes after test/EmbeddingSpMDMNBitTest.cc:21-46 (batch, rows, dim, average length)
  const int shapes[][4] = {{10, 400, 2, 5}, {10, 400, 4, 5}, {10, 400, 8, 5}, {10, 400, 40, 5}, {10, 400, 48, 5},
                           {10, 400, 56, 5}, {3, 1000, 86, 20}, {10, 400, 128, 5}, {10, 400, 164, 5}, {100, 4000, 256, 20}};
  unsigned seed = 1;
  for (auto& s : shapes)
    for (int bit_rate : {2, 4})
      for (int weighted = 0; weighted < 2; ++weighted)
        for (int normalize = 0; normalize < 2; ++normalize)
          for (int corner = 0; corner < 4; ++corner) {
            if (bit_rate == 2 && s[2] % 4) continue;
            run_nbit<int64_t, int32_t, float>(bit_rate, s[2], s[0], s[1], s[3], weighted, normalize, true, corner, ++seed);
            const bool offsets_form = corner != 3 && (seed & 1);
            run_nbit<int32_t, int64_t, fbgemm_amd::float16>(bit_rate, s[2], s[0], s[1], s[3], weighted, normalize,
                                                            offsets_form, corner, ++seed);
          }
  for (auto& s : shapes)
    for (int weighted = 0; weighted < 2; ++weighted)
      for (int normalize = 0; normalize < 2; ++normalize) {
        run_8bit<int64_t, int32_t>(s[2], s[0], s[1], s[3], weighted, normalize, ++seed);
        run_8bit<int32_t, int32_t>(s[2], s[0], s[1], s[3], weighted, normalize, ++seed);
      }
  for (int D : {2, 8, 40, 86, 128, 256}) {
    run_no_bag_and_fp8<int64_t>(D, 77, 300, ++seed);
    run_no_bag_and_fp8<int32_t>(D, 500, 1000, ++seed);
  }
  for (int weighted = 0; weighted < 2; ++weighted) {
    run_remap<int32_t>(10, 400, 5, weighted, ++seed);
    run_remap<int64_t>(1000, 4000, 20, weighted, ++seed);
  }
  for (int cols : {4, 8, 64, 100, 128, 260})
    for (int rows : {1, 7, 130}) run_quantizers(rows, cols, ++seed);
  run_fixed_numbers();
  // Kernels called from several host threads at once, each on a stream of its own, as the
  // reference's generated kernels may be: every thread mixes calls that succeed with calls
  // that must return false (out-of-range index, unmatched lengths), lengths as well as offsets.
  {
    std::vector<std::thread> threads;
    for (int th = 0; th < 4; ++th)
      threads.emplace_back([th] {
        hipStream_t stream;
        if (hipStreamCreate(&stream) != hipSuccess) { ++failures; return; }
        fbgemm_amd::set_stream(stream);
        unsigned seed = 5000 + 1000 * th;
        for (int it = 0; it < 12; ++it)
          for (int corner = 0; corner < 4; ++corner) {
            run_nbit<int64_t, int32_t, float>(4, 128, 10 + th, 400, 5, it & 1, it & 2, (it + th) & 1 || corner == 3 ? true : false,
                                              corner, ++seed);
            run_8bit<int32_t, int64_t>(64, 20, 300, 6, it & 1, it & 2, ++seed);
          }
        fbgemm_amd::set_stream(nullptr);
        (void)hipStreamSynchronize(stream);
        (void)hipStreamDestroy(stream);
      });
    for (auto& t : threads) t.join();
  }
  printf("%s: %d failure(s)\n", failures ? "FAILED" : "PASSED", failures.load());
  return failures ? 1 : 0;
}
