/* Benchmarks and tests only. Nothing declared here has a counterpart in the
 * reference and nothing here is part of the drop-in boundary
 * (include/fbgemm_amd.h): yardstick kernels for profiles, and the switches the
 * A/B measurements and the parity tests use to steer the library.
 *
 * fbgemm_amd_bench_* live in a library of their own, libfbgemm_amd_bench.so
 * (fbgemm_amd/csrc/bench_kernels.hip); the switches are part of libfbgemm_amd.so
 * because they reach into it. */
#ifndef FBGEMM_AMD_BENCH_H_
#define FBGEMM_AMD_BENCH_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

struct fbgemm_amd_tbe_plan;

/* ---- libfbgemm_amd_bench.so: 0 on success, negative on error ------------------ */
const char* fbgemm_amd_bench_last_error(void);

/* A plain device-to-device copy of `bytes` (a multiple of 16) by a kernel named
 * calibration_copy_kernel: profiles scale the hardware byte counters of the
 * lookup kernels against what the same counters read for this copy. */
int fbgemm_amd_bench_calibration_copy(const void* d_src, void* d_dst, int64_t bytes, void* stream);

/* Every lane reads 16 bytes per load, 8 loads in flight, through `bytes` of d_src
 * once (kernel stream_read_kernel). d_sink: at least 8192 dwords. */
int fbgemm_amd_bench_stream_read(const void* d_src, int64_t bytes, void* d_sink, int64_t sink_dwords, void* stream);

/* `n` rows d_rows[i] (int32; clamped to 0 .. rows - 1) of a table whose rows are
 * row_stride bytes apart; lanes_per_row consecutive lanes read 16 bytes each from
 * byte_offset on (4 = what rows with a 4-byte header in front of their data give:
 * loads at 4-byte alignment); `waves` workgroups of one wave each; d_sink holds
 * sink_dwords >= waves dwords. mode: how the rows are fetched. */
enum {
  FBGEMM_AMD_BENCH_GATHER_REGISTERS = 0,    /* 8 rows per lane group in flight, into registers (gather_lines_kernel<8>) */
  FBGEMM_AMD_BENCH_GATHER_REGISTERS_16 = 1, /* 16 rows in flight */
  FBGEMM_AMD_BENCH_GATHER_LDS = 2,          /* 8 rows in flight, 16-byte loads that write LDS directly (gather_lines_lds_kernel) */
};
int fbgemm_amd_bench_gather(const void* d_table, int64_t rows, int64_t row_stride, int32_t lanes_per_row, int32_t byte_offset,
                            const int32_t* d_rows, int64_t n, void* d_sink, int64_t sink_dwords, int32_t waves, int32_t mode,
                            void* stream);

/* ---- libfbgemm_amd.so: process-wide switches ----------------------------------- *
 * Results are bit-identical under every setting. Not synchronised: set them while
 * no other thread is inside the library.
 * fbgemm_amd_set_lean: 1 = shapes the lean kernel takes go to it (the default,
 * also FBGEMM_AMD_LEAN in the environment at load time), 0 = everything goes
 * through the general kernel, -1 = back to the default.
 * fbgemm_amd_set_narrow_below_waves: launches of fewer waves than this take
 * 4-byte lanes (default 1024, FBGEMM_AMD_NARROW_BELOW_WAVES at load time; -1 =
 * back to the default).
 * fbgemm_amd_set_wide4: which lean kernel large forwards take whose lean tables
 * all have 4-bit rows in bags of 8 lanes and more: 0 = the general-purpose one,
 * 2 = the four-waves-per-SIMD instance, 1 = whichever the first forwards of a
 * batch size measure as the faster (the default, FBGEMM_AMD_WIDE4 at load
 * time), -1 = back to the default. */
int fbgemm_amd_set_lean(int32_t on);
int fbgemm_amd_set_narrow_below_waves(int32_t waves);
int fbgemm_amd_set_wide4(int32_t mode);

/* Timing of the lookup kernels alone: while `on` is 1, forwards of the plan skip
 * the bag scheduler and take the bag order the last forward on the same stream
 * left behind (valid as long as the offsets are the same), so a run of forwards
 * is the lookup kernels back to back and a pair of events around the run gives
 * their average duration. 0 switches it off. */
int fbgemm_amd_tbe_plan_reuse_order(struct fbgemm_amd_tbe_plan* plan, int32_t on);

#ifdef __cplusplus
}
#endif
#endif /* FBGEMM_AMD_BENCH_H_ */
