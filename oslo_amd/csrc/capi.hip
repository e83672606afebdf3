// Process-wide pieces of the C ABI: error strings, tuning knobs, device
// facts and workspace sizing.
#include "capi.h"

#include <string.h>

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

Tuning g_tune = {0, 0, 0, 0, 0, 0, 0, 0, 0};

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
  struct Entry {
    const char *name;
    int *slot;
  };
  const Entry table[] = {
      {"norm_fwd_vpl", &oslo::g_tune.norm_fwd_vpl},
      {"norm_bwd_vpl", &oslo::g_tune.norm_bwd_vpl},
      {"norm_bwd_blocks_per_cu", &oslo::g_tune.norm_bwd_blocks_per_cu},
      {"softmax_rows_per_wave", &oslo::g_tune.softmax_rows_per_wave},
      {"softmax_lanes_per_row", &oslo::g_tune.softmax_lanes_per_row},
      {"softmax_fwd_elems", &oslo::g_tune.softmax_fwd_elems},
      {"norm_lanes_per_row", &oslo::g_tune.norm_lanes_per_row},
      {"eltwise_tile_max", &oslo::g_tune.eltwise_tile_max},
      {"eltwise_tile_min", &oslo::g_tune.eltwise_tile_min},
      {"eltwise_unroll", &oslo::g_tune.eltwise_unroll},
      {"eltwise_rowgroups", &oslo::g_tune.eltwise_rowgroups},
      {"eltwise_fwd_steps", &oslo::g_tune.eltwise_fwd_steps},
      {"norm_bwd_waves", &oslo::g_tune.norm_bwd_waves},
      {"norm_fwd_waves", &oslo::g_tune.norm_fwd_waves},
      {"norm_bwd_prefetch", &oslo::g_tune.norm_bwd_prefetch},
      {"norm_fwd_iters", &oslo::g_tune.norm_fwd_iters},
      {"adam_unroll", &oslo::g_tune.adam_unroll},
  };
  for (const Entry &e : table) {
    if (strcmp(e.name, key) == 0) {
      *e.slot = value;
      return OSLO_OK;
    }
  }
  return oslo::fail(OSLO_ERR_INVALID_ARGUMENT, "tune: unknown key '%s'", key);
}

}  // extern "C"
