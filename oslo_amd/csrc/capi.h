// Host-side helpers shared by the C-ABI entry points: error reporting,
// argument checks, launch-heuristic knobs and cached device facts.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/oslo_hip.h"
#include "../../include/oslo_hip_testing.h"

namespace oslo {

// Records the calling thread's error message and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// hipGetLastError() after a launch -> OSLO_OK or OSLO_ERR_LAUNCH.
int check_launch(const char *what);

// Device pointer to {seed, offset} that the *_rng entry points put in place
// for the duration of their call on the calling thread (null otherwise).
const uint64_t *current_rng_state();
void set_current_rng_state(const uint64_t *state);

// Number of compute units of the current device (cached per device id).
int device_cu_count();

// Launch-heuristic overrides set through oslo_tune(); 0 = use the default.
struct Tuning {
  int norm_fwd_vpl;
  int norm_bwd_vpl;
  int norm_bwd_blocks_per_cu;
  int softmax_rows_per_wave;
  int softmax_lanes_per_row;
  int softmax_fwd_elems;
  int softmax_rows_per_block;
  int norm_lanes_per_row;
  int eltwise_tile_max;
  int eltwise_tile_min;
  int eltwise_unroll;
  int eltwise_rowgroups;
  int eltwise_fwd_steps;
  int norm_bwd_waves;
  int norm_fwd_waves;
  int norm_bwd_prefetch;
  int norm_fwd_iters;
  int adam_unroll;
  int softmax_bias_order;
  int colsum_defer;
  int softmax_causal_order;
  int softmax_bias_group;
  int colsum_slices;
};
// oslo_tune() writes a process-wide table under a lock; every entry point
// copies that table into a per-thread snapshot before it plans a launch
// (tune_snapshot()), and the launch code reads only the snapshot: a sweep
// that changes a knob on another thread cannot change a launch half way.
extern thread_local Tuning t_tune;
void tune_snapshot();
#define g_tune (::oslo::t_tune)

inline bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

inline bool valid_dtype(int d) {
  return d == OSLO_DTYPE_F32 || d == OSLO_DTYPE_F16 || d == OSLO_DTYPE_BF16;
}

inline int dtype_size(int d) {
  return d == OSLO_DTYPE_F64 ? 8 : d == OSLO_DTYPE_F32 ? 4 : 2;
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// A dispatch carries its size as a 32-bit count of work-items, so workgroups x
// workgroup size must stay below 2^32.  The runtime does not report an excess:
// the count wraps and only part of the grid runs.  Launchers therefore cap the
// grid of a kernel that strides over its work, and split the work of a kernel
// that does one unit per workgroup into several launches.
inline int64_t max_workgroups(int threads) { return (int64_t)0xffffffffll / threads; }

// Double-precision LayerNorm / RMSNorm (norm_f64.hip); every pointer is to
// double data.
int launch_norm_f64_fwd(bool rms, const void *x, const void *gamma,
                        const void *beta, void *y, void *mean, void *invvar,
                        int64_t n1, int64_t n2, double eps, hipStream_t st);
int launch_norm_f64_bwd(bool rms, const void *dy, const void *x,
                        const void *mean, const void *invvar,
                        const void *gamma, void *dx, void *dgamma, void *dbeta,
                        int64_t n1, int64_t n2, hipStream_t st);

// Column-partial workspace layout shared by the backward kernels and the
// finalize kernel: `narrays` fp32 arrays of [parts, cols].
int64_t colsum_parts_norm(int64_t n1, int64_t n2);
int64_t colsum_parts_eltwise(int64_t rows, int64_t cols);

}  // namespace oslo

#define OSLO_REQUIRE(cond, ...)                                       \
  do {                                                                \
    if (!(cond)) return ::oslo::fail(OSLO_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)
