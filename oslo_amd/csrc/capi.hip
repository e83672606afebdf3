// Process-wide pieces of the C ABI: error strings, tuning knobs, device
// facts and workspace sizing.
#include "capi.h"

#include <string.h>

#include <mutex>

namespace oslo {

static thread_local char t_err[512] = "";
static thread_local const uint64_t *t_rng_state = nullptr;

const uint64_t *current_rng_state() { return t_rng_state; }
void set_current_rng_state(const uint64_t *state) { t_rng_state = state; }

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(t_err, sizeof(t_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  const hipError_t e = hipGetLastError();
  if (e == hipSuccess) return OSLO_OK;
  return fail(OSLO_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

int device_cu_count() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) !=
            hipSuccess ||
        n <= 0)
      n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

static Tuning s_tune_shared = {};  // all zero: every heuristic at its built-in choice
static std::mutex s_tune_lock;
thread_local Tuning t_tune = {};

void tune_snapshot() {
  std::lock_guard<std::mutex> guard(s_tune_lock);
  t_tune = s_tune_shared;
}

}  // namespace oslo

extern "C" {

int oslo_rng_from_device(const uint64_t *state) {
  oslo::set_current_rng_state(state);
  return OSLO_OK;
}

const char *oslo_hip_last_error(void) { return oslo::t_err; }

const char *oslo_hip_arch(void) { return "gfx950"; }

int oslo_hip_abi_version(void) { return OSLO_HIP_ABI_VERSION; }

int64_t oslo_workspace_bytes(int op, int64_t n1, int64_t n2) {
  oslo::tune_snapshot();
  if (n1 < 0 || n2 < 1) {
    oslo::fail(OSLO_ERR_INVALID_ARGUMENT, "workspace_bytes: bad shape");
    return OSLO_ERR_INVALID_ARGUMENT;
  }
  if (n1 == 0) return 0;
  switch (op) {
    case OSLO_OP_LN_BWD:
      return 2 * oslo::colsum_parts_norm(n1, n2) * n2 * (int64_t)sizeof(float);
    case OSLO_OP_BIAS_DROPOUT_ADD_NORM_BWD:
      return 3 * oslo::colsum_parts_norm(n1, n2) * n2 * (int64_t)sizeof(float);
    case OSLO_OP_RMS_BWD:
      return oslo::colsum_parts_norm(n1, n2) * n2 * (int64_t)sizeof(float);
    case OSLO_OP_BIAS_GELU_BWD:
    case OSLO_OP_BIAS_DROPOUT_ADD_BWD:
      return oslo::colsum_parts_eltwise(n1, n2) * n2 * (int64_t)sizeof(float);
    default:
      oslo::fail(OSLO_ERR_INVALID_ARGUMENT, "workspace_bytes: unknown op %d", op);
      return OSLO_ERR_INVALID_ARGUMENT;
  }
}

int oslo_tune(const char *key, int value) {
  if (key == nullptr || value < 0)
    return oslo::fail(OSLO_ERR_INVALID_ARGUMENT, "tune: bad arguments");
  // 0 restores the built-in choice; any other value must be one the launch
  // code has a kernel build and a valid workgroup shape for
  enum Kind { kPow2, kRange, kLanes, kPow2or3 };
  struct Entry {
    const char *name;
    int *slot;
    Kind kind;
    int lo, hi;  // kPow2: powers of two in [lo, hi]; kRange: lo..hi
  };
  std::lock_guard<std::mutex> guard(oslo::s_tune_lock);
  oslo::Tuning &shared = oslo::s_tune_shared;
  const Entry table[] = {
      {"norm_fwd_vpl", &shared.norm_fwd_vpl, kPow2or3, 1, 8},
      {"norm_bwd_vpl", &shared.norm_bwd_vpl, kPow2, 1, 4},
      {"norm_bwd_blocks_per_cu", &shared.norm_bwd_blocks_per_cu, kRange, 1, 8},
      {"softmax_rows_per_wave", &shared.softmax_rows_per_wave, kPow2, 1, 4},
      {"softmax_lanes_per_row", &shared.softmax_lanes_per_row, kLanes, 1, 64},
      {"softmax_fwd_elems", &shared.softmax_fwd_elems, kPow2, 16, 64},
      {"softmax_rows_per_block", &shared.softmax_rows_per_block, kRange, 1, 16},
      {"norm_lanes_per_row", &shared.norm_lanes_per_row, kLanes, 8, 64},
      {"eltwise_tile_max", &shared.eltwise_tile_max, kPow2, 1, 256},
      {"eltwise_tile_min", &shared.eltwise_tile_min, kPow2, 1, 256},
      {"eltwise_unroll", &shared.eltwise_unroll, kPow2, 1, 8},
      {"eltwise_rowgroups", &shared.eltwise_rowgroups, kRange, 1, 4096},
      {"eltwise_fwd_steps", &shared.eltwise_fwd_steps, kRange, 1, 64},
      {"norm_bwd_waves", &shared.norm_bwd_waves, kRange, 1, 16},
      {"norm_fwd_waves", &shared.norm_fwd_waves, kRange, 1, 16},
      {"norm_bwd_prefetch", &shared.norm_bwd_prefetch, kRange, 1, 2},
      {"norm_fwd_iters", &shared.norm_fwd_iters, kRange, 1, 16},
      {"adam_unroll", &shared.adam_unroll, kPow2, 1, 4},
      {"softmax_bias_order", &shared.softmax_bias_order, kRange, 1, 3},
      {"colsum_defer", &shared.colsum_defer, kRange, 1, 1},
      {"softmax_causal_order", &shared.softmax_causal_order, kRange, 1, 3},
      {"softmax_bias_group", &shared.softmax_bias_group, kPow2, 1, 256},
      {"colsum_slices", &shared.colsum_slices, kPow2, 64, 256},
  };
  for (const Entry &e : table) {
    if (strcmp(e.name, key) == 0) {
      bool ok = value == 0;
      if (!ok && value >= e.lo && value <= e.hi) {
        const bool pow2 = (value & (value - 1)) == 0;
        ok = e.kind == kRange || (e.kind == kPow2 && pow2) || (e.kind == kPow2or3 && (pow2 || value == 3)) ||
             (e.kind == kLanes && (value == 1 || (pow2 && value >= 8)));
      }
      if (!ok)
        return oslo::fail(OSLO_ERR_INVALID_ARGUMENT,
                          "tune: %d is no valid value for '%s'", value, key);
      *e.slot = value;
      return OSLO_OK;
    }
  }
  return oslo::fail(OSLO_ERR_INVALID_ARGUMENT, "tune: unknown key '%s'", key);
}

}  // extern "C"
