// Expert placement on the MoE path: the static tables of a placement pattern (host code) and the two
// device operations the layer runs per step when a placement is in use: the remap of routed expert
// ids to deployed positions and the per-expert activation counters.
//
// Reference: omni/accelerators/placement/omni_planner/cpp/placement_mapping.cpp:223-257 (positions),
// :374-427 (selector), omni/accelerators/placement/omni_planner/omni_planner.py:244-274 (plan = a table
// lookup on the ids), :337-343 (record_activation).
#include "common.h"

#include <algorithm>

namespace {

struct RemapArgs {
  const int32_t* ids;
  int64_t n;
  const int32_t* map;
  int n_map;
  int32_t* out;
};

__global__ void __launch_bounds__(256) remap_ids_kernel(RemapArgs a) {
  // the table is small (one entry per logical expert): it stays in the L1/L2 and the lookups coalesce on the ids
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n; i += stride) {
    const int32_t e = a.ids[i];
    a.out[i] = ((uint32_t)e < (uint32_t)a.n_map) ? a.map[e] : e;
  }
}

__global__ void __launch_bounds__(256) record_activation_kernel(int64_t* counts, const int32_t* tokens, int n, int64_t modulus) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counts[i] = (counts[i] + (int64_t)tokens[i]) % modulus;
}

}  // namespace

extern "C" int omni_placement_tables(const int32_t* pattern, int world, int layers, int experts, int rank,
                                     int devices_per_host, int num_deploy, int32_t* position_to_expert,
                                     int32_t* selector) {
  // host code on host arrays (host_logic.h)
  return omni_host::placement_tables(pattern, world, layers, experts, rank, devices_per_host, num_deploy,
                                     position_to_expert, selector);
}

extern "C" int omni_moe_remap_ids(const int32_t* ids, int64_t n, const int32_t* map, int n_map, int32_t* out, void* stream) {
  if (n < 0 || n_map <= 0) OMNI_FAIL(OMNI_E_INVALID, "remap_ids: bad sizes n=%lld n_map=%d", (long long)n, n_map);
  if (n == 0) return OMNI_OK;
  if (!ids || !map || !out) OMNI_FAIL(OMNI_E_INVALID, "remap_ids: null pointer");
  RemapArgs a{ids, n, map, n_map, out};
  const unsigned blocks = (unsigned)std::min<int64_t>((n + 255) / 256, 2048);
  hipLaunchKernelGGL(remap_ids_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
  OMNI_CHECK_LAUNCH("remap_ids");
  return OMNI_OK;
}

extern "C" int omni_moe_record_activation(int64_t* counts, const int32_t* tokens_per_expert, int n, int64_t modulus, void* stream) {
  if (n < 0 || modulus <= 0) OMNI_FAIL(OMNI_E_INVALID, "record_activation: bad sizes n=%d modulus=%lld", n, (long long)modulus);
  if (n == 0) return OMNI_OK;
  if (!counts || !tokens_per_expert) OMNI_FAIL(OMNI_E_INVALID, "record_activation: null pointer");
  hipLaunchKernelGGL(record_activation_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, counts, tokens_per_expert, n, modulus);
  OMNI_CHECK_LAUNCH("record_activation");
  return OMNI_OK;
}
