// Expert placement on the MoE path: the static tables of a placement pattern (host code) and the two
// device operations the layer runs per step when a placement is in use: the remap of routed expert
// ids to deployed positions and the per-expert activation counters.
//
// Reference: omni/accelerators/placement/omni_planner/cpp/placement_mapping.cpp:223-257 (positions),
// :374-427 (selector), omni/accelerators/placement/omni_planner/omni_planner.py:244-274 (plan = a table
// lookup on the ids), :337-343 (record_activation).
#include "common.h"

#include <vector>

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
  if (!pattern || !selector) OMNI_FAIL(OMNI_E_INVALID, "placement_tables: null pointer");
  if (world < 1 || layers < 1 || experts < 1 || devices_per_host < 1)
    OMNI_FAIL(OMNI_E_INVALID, "placement_tables: bad sizes world=%d layers=%d experts=%d devices_per_host=%d", world, layers, experts, devices_per_host);
  if (rank < 0 || rank >= world) OMNI_FAIL(OMNI_E_INVALID, "placement_tables: rank %d outside [0,%d)", rank, world);
  if (num_deploy < experts || num_deploy % world != 0)
    OMNI_FAIL(OMNI_E_INVALID, "placement_tables: %d deployed positions for %d experts on %d devices", num_deploy, experts, world);
  const int per_device = num_deploy / world;
  // positions: device r owns [r*per_device, (r+1)*per_device); its deployed experts take them in id order
  std::vector<int32_t> pos((size_t)layers * num_deploy, -1);
  std::vector<int32_t> copies((size_t)layers * experts, 0);
  for (int l = 0; l < layers; ++l)
    for (int r = 0; r < world; ++r) {
      int local = 0;
      for (int e = 0; e < experts; ++e) {
        const int32_t v = pattern[((size_t)r * layers + l) * experts + e];
        if (v != 0 && v != 1) OMNI_FAIL(OMNI_E_INVALID, "placement_tables: pattern[%d][%d][%d] = %d is neither 0 nor 1", r, l, e, v);
        if (v == 0) continue;
        if (local >= per_device)
          OMNI_FAIL(OMNI_E_INVALID, "placement_tables: device %d deploys more than %d experts in layer %d", r, per_device, l);
        pos[(size_t)l * num_deploy + (size_t)r * per_device + local] = e;
        copies[(size_t)l * experts + e]++;
        ++local;
      }
    }
  // selector: for each logical expert the position this rank sends its tokens to: the copy on the rank itself, else
  // one of the copies on the rank's host, else one of the others, each set shared out by rank modulo its size
  const int my_host = rank / devices_per_host;
  std::vector<int32_t> same, far;
  for (int l = 0; l < layers; ++l)
    for (int e = 0; e < experts; ++e) {
      same.clear();
      far.clear();
      int32_t own = -1;
      for (int p = 0; p < num_deploy; ++p) {
        if (pos[(size_t)l * num_deploy + p] != e) continue;
        const int dev = p / per_device;
        if (dev == rank) { if (own < 0) own = p; }
        else if (dev / devices_per_host == my_host) same.push_back(p);
        else far.push_back(p);
      }
      int32_t s = 0;  // an expert that is deployed nowhere keeps position 0, as in the reference's zero-filled table
      if (own >= 0) s = own;
      else if (!same.empty()) s = same[rank % same.size()];
      else if (!far.empty()) s = far[rank % far.size()];
      selector[(size_t)l * experts + e] = s;
    }
  if (position_to_expert)
    for (size_t i = 0; i < pos.size(); ++i) position_to_expert[i] = pos[i];
  return OMNI_OK;
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
