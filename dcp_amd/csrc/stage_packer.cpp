// Stage packer of the planner: which attention blocks ("workloads") each device may run in the
// next pipeline stage, and which data blocks have to be sent to it first.  Host code only; it is
// in this library because it is the one natively compiled routine of the reference planner
// (csrc/pipeline_generator/pipeline_generator.cpp:19-323, bound as dcp_cpp.greedy_selection_per_device
// and called once per stage from dcp/core/pipeline.py:651-666,703-716).
//
// The reference keeps devices, pending workloads and "which device holds which block since which
// stage" in hash sets and maps of tuples.  Here everything is dense and indexed: devices are
// 0..n_devices-1 in the caller's order, the holder table is one int32 per (device, block), the
// per-device pending lists are sorted once.  Where the reference's result depends on the iteration
// order of a hash table (ties), this routine takes the FIRST candidate in index order:
//   - several devices with the same accumulated compute time: the lowest device index goes first;
//   - several holders of a block with the same outgoing load: the lowest device index sends;
//   - workloads of equal cost: the lower workload id is tried first.
// Loads, sizes and costs are accumulated in float, in the reference's order.
#include <algorithm>
#include <cfloat>
#include <cstdint>
#include <vector>

#include "common.h"

namespace {

struct Packer {
  int n_devices, n_inputs;
  const int32_t* node;           // [n_devices]
  const float* input_sizes;      // [n_inputs]
  const uint8_t* kind;           // [n_inputs] DCP_BLOCK_*
  const float* target;           // [n_devices] cap on a device's outgoing cross-node bytes
  int32_t* local;                // [n_devices * n_inputs] stage since which the block is held, or DCP_NOT_HELD
  bool is_bw;
  int stage_id;
  std::vector<float> cross_load, intra_load;

  // one (block, source) decision of a feasibility check
  struct Need {
    int input, src;
    bool cross;
  };
  std::vector<Need> needs;
  std::vector<float> cross_add, intra_add;  // bytes this check would add per source device
  std::vector<int> touched_cross, touched_intra;  // the devices with an entry in cross_add / intra_add
  std::vector<char> in_cross, in_intra;

  bool held(int d, int input) const { return local[(size_t)d * n_inputs + input] != DCP_NOT_HELD; }

  // Sources for the blocks of `inputs` that device `dst` lacks; false if some source's cross-node
  // budget would be exceeded.  A block may only be taken from a device that held it before this
  // stage; a holder on dst's node is preferred (least loaded first), else the least loaded remote one.
  // Returns -1 if nobody can supply a block.
  int check(const int32_t* inputs, int n, int dst) {
    needs.clear();
    for (int d : touched_cross) cross_add[d] = 0.0f, in_cross[d] = 0;
    for (int d : touched_intra) intra_add[d] = 0.0f, in_intra[d] = 0;
    touched_cross.clear();
    touched_intra.clear();
    for (int i = 0; i < n; ++i) {
      const int input = inputs[i];
      if (held(dst, input)) continue;
      int best_near = -1, best_far = -1;
      for (int d = 0; d < n_devices; ++d) {
        const int32_t since = local[(size_t)d * n_inputs + input];
        if (since == DCP_NOT_HELD || since >= stage_id) continue;
        if (node[d] == node[dst]) {
          if (best_near < 0 || intra_load[d] < intra_load[best_near]) best_near = d;
        } else {
          if (best_far < 0 || cross_load[d] < cross_load[best_far]) best_far = d;
        }
      }
      // the gradient of the output travels with the output in a backward plan: count it
      const float bytes = input_sizes[input];
      const bool twice = kind[input] == DCP_BLOCK_OUT && is_bw;
      if (best_near >= 0) {
        needs.push_back({input, best_near, false});
        if (!in_intra[best_near]) in_intra[best_near] = 1, touched_intra.push_back(best_near);
        if (twice) intra_add[best_near] += bytes;
        intra_add[best_near] += bytes;
      } else if (best_far >= 0) {
        needs.push_back({input, best_far, true});
        if (!in_cross[best_far]) in_cross[best_far] = 1, touched_cross.push_back(best_far);
        if (twice) cross_add[best_far] += bytes;
        cross_add[best_far] += bytes;
      } else {
        return -1;
      }
    }
    for (int d : touched_cross)
      if (cross_load[d] + cross_add[d] > target[d]) return 0;
    return 1;
  }
};

}  // namespace

extern "C" int dcp_greedy_stage_selection(
    int n_devices, const int32_t* device_node, int n_workloads, const float* workload_costs,
    const uint8_t* workload_scheduled, int n_inputs, const float* input_sizes, const uint8_t* input_kind,
    const int32_t* workload_input_offsets, const int32_t* workload_inputs,
    const int32_t* device_workload_offsets, const int32_t* device_workloads, int32_t* held_since,
    const float* target_cross_node_load, int is_bw, int stage_id, int32_t* unlocked_by,
    int32_t* comm_dst, int32_t* comm_input, int32_t* comm_src, int64_t comm_capacity, int64_t* n_comm,
    float* cross_node_load_out, float* intra_node_load_out) {
  using namespace dcp;
  DCP_REQUIRE(n_devices > 0 && n_workloads >= 0 && n_inputs >= 0, "stage_selection: sizes must be non-negative (devices: positive)");
  DCP_REQUIRE(device_node && workload_input_offsets && device_workload_offsets && held_since &&
                  target_cross_node_load && unlocked_by && n_comm,
              "stage_selection: null argument");
  DCP_REQUIRE(n_workloads == 0 || (workload_costs && workload_scheduled), "stage_selection: null workload tables");
  DCP_REQUIRE(n_inputs == 0 || (input_sizes && input_kind), "stage_selection: null block tables");
  DCP_REQUIRE(comm_capacity >= 0 && (comm_capacity == 0 || (comm_dst && comm_input && comm_src)),
              "stage_selection: null transfer list");
  DCP_REQUIRE(workload_input_offsets[0] == 0 && device_workload_offsets[0] == 0, "stage_selection: offsets must start at 0");
  for (int w = 0; w < n_workloads; ++w)
    DCP_REQUIRE(workload_input_offsets[w + 1] >= workload_input_offsets[w], "stage_selection: workload_input_offsets must not decrease");
  for (int d = 0; d < n_devices; ++d)
    DCP_REQUIRE(device_workload_offsets[d + 1] >= device_workload_offsets[d], "stage_selection: device_workload_offsets must not decrease");
  DCP_REQUIRE(workload_input_offsets[n_workloads] == 0 || workload_inputs, "stage_selection: null workload_inputs");
  DCP_REQUIRE(device_workload_offsets[n_devices] == 0 || device_workloads, "stage_selection: null device_workloads");
  for (int i = 0; i < workload_input_offsets[n_workloads]; ++i)
    DCP_REQUIRE(workload_inputs[i] >= 0 && workload_inputs[i] < n_inputs, "stage_selection: block id %d out of range", workload_inputs[i]);
  for (int i = 0; i < device_workload_offsets[n_devices]; ++i)
    DCP_REQUIRE(device_workloads[i] >= 0 && device_workloads[i] < n_workloads, "stage_selection: workload id %d out of range",
                device_workloads[i]);
  for (int i = 0; i < n_inputs; ++i)
    DCP_REQUIRE(input_kind[i] <= DCP_BLOCK_DOUT, "stage_selection: block kind %d unknown", (int)input_kind[i]);

  Packer pk;
  pk.n_devices = n_devices;
  pk.n_inputs = n_inputs;
  pk.node = device_node;
  pk.input_sizes = input_sizes;
  pk.kind = input_kind;
  pk.target = target_cross_node_load;
  pk.local = held_since;
  pk.is_bw = is_bw != 0;
  pk.stage_id = stage_id;
  pk.cross_load.assign(n_devices, 0.0f);
  pk.intra_load.assign(n_devices, 0.0f);
  pk.cross_add.assign(n_devices, 0.0f);
  pk.intra_add.assign(n_devices, 0.0f);
  pk.in_cross.assign(n_devices, 0);
  pk.in_intra.assign(n_devices, 0);

  // The out / lse / dout blocks of a workload (at most one each): the three travel together,
  // priced and placed through the out block.
  struct Trio {
    int out = -1, lse = -1, dout = -1;
  };
  auto trio_of = [&](int w) {
    Trio t;
    for (int i = workload_input_offsets[w]; i < workload_input_offsets[w + 1]; ++i) {
      const int input = workload_inputs[i];
      if (input_kind[input] == DCP_BLOCK_OUT) t.out = input;
      else if (input_kind[input] == DCP_BLOCK_LSE) t.lse = input;
      else if (input_kind[input] == DCP_BLOCK_DOUT) t.dout = input;
    }
    return t;
  };
  for (int w = 0; w < n_workloads; ++w) {
    const Trio t = trio_of(w);
    DCP_REQUIRE((t.out < 0) == (t.lse < 0), "stage_selection: workload %d has an out block without its lse block (or the reverse)", w);
    DCP_REQUIRE(t.dout < 0 || t.out >= 0, "stage_selection: workload %d has a dout block without an out block", w);
  }

  // pending workloads per device, most expensive first (equal cost: lower id first)
  std::vector<std::vector<int>> pending(n_devices);
  for (int d = 0; d < n_devices; ++d) {
    auto& list = pending[d];
    for (int i = device_workload_offsets[d]; i < device_workload_offsets[d + 1]; ++i)
      if (!workload_scheduled[device_workloads[i]]) list.push_back(device_workloads[i]);
    std::sort(list.begin(), list.end());
    list.erase(std::unique(list.begin(), list.end()), list.end());
    std::stable_sort(list.begin(), list.end(), [&](int a, int b) { return workload_costs[a] > workload_costs[b]; });
  }
  for (int w = 0; w < n_workloads; ++w) unlocked_by[w] = -1;

  int64_t count = 0;
  bool overflow = false;
  auto emit = [&](int dst, int input, int src) {
    if (count < comm_capacity) {
      comm_dst[count] = dst;
      comm_input[count] = input;
      comm_src[count] = src;
    } else {
      overflow = true;
    }
    ++count;
  };
  // record the transfers of the last successful check, cross-node ones first, and book their bytes
  auto commit = [&](int dst, const Trio& t) {
    for (int pass = 0; pass < 2; ++pass)
      for (const auto& need : pk.needs) {
        if (need.cross != (pass == 0)) continue;
        emit(dst, need.input, need.src);
        if (need.input == t.out) {
          emit(dst, t.lse, need.src);
          if (t.dout >= 0) emit(dst, t.dout, need.src);
        }
      }
    for (int d : pk.touched_cross) pk.cross_load[d] += pk.cross_add[d];
    for (int d : pk.touched_intra) pk.intra_load[d] += pk.intra_add[d];
  };

  // ---- phase 1: the device with the least compute so far gets its most expensive workload whose
  // missing blocks fit the senders' budgets; stop at the first device that cannot take any --------
  std::vector<float> ready_time(n_devices, 0.0f);
  std::vector<char> done(n_devices, 0);
  int n_done = 0;
  std::vector<int32_t> wanted;
  while (n_done < n_devices) {
    int dev = -1;
    float least = FLT_MAX;
    for (int d = 0; d < n_devices; ++d)
      if (!done[d] && ready_time[d] < least) {
        least = ready_time[d];
        dev = d;
      }
    if (dev < 0) break;  // every remaining device has an unrepresentably large time
    auto& list = pending[dev];
    if (list.empty()) {
      done[dev] = 1;
      ++n_done;
      continue;
    }
    bool progress = false;
    for (size_t at = 0; at < list.size(); ++at) {
      const int w = list[at];
      const Trio t = trio_of(w);
      wanted.clear();
      for (int i = workload_input_offsets[w]; i < workload_input_offsets[w + 1]; ++i) {
        const int input = workload_inputs[i];
        if (input != t.out && input != t.lse && input != t.dout) wanted.push_back(input);
      }
      if (t.out >= 0) wanted.push_back(t.out);
      const int ok = pk.check(wanted.data(), (int)wanted.size(), dev);
      if (ok < 0) return fail(DCP_ERR_ARG, "stage_selection: no device held a block of workload %d before stage %d", w, stage_id);
      if (!ok) continue;
      unlocked_by[w] = dev;
      commit(dev, t);
      for (int i = workload_input_offsets[w]; i < workload_input_offsets[w + 1]; ++i) {
        int32_t& since = held_since[(size_t)dev * n_inputs + workload_inputs[i]];
        if (since == DCP_NOT_HELD) since = stage_id;
      }
      ready_time[dev] += workload_costs[w];
      list.erase(list.begin() + at);
      progress = true;
      break;
    }
    if (!progress) break;
  }

  // ---- phase 2: with what is left of the budgets, send blocks of the still pending workloads
  // ahead of their stage, device by device, most expensive workload first ---------------------------
  for (int dev = 0; dev < n_devices; ++dev)
    for (int w : pending[dev]) {
      const Trio t = trio_of(w);
      for (int i = workload_input_offsets[w]; i < workload_input_offsets[w + 1]; ++i) {
        const int32_t input = workload_inputs[i];
        if (input == t.lse || input == t.dout) continue;
        if (pk.held(dev, input)) continue;
        const int ok = pk.check(&input, 1, dev);
        if (ok < 0) return fail(DCP_ERR_ARG, "stage_selection: no device held block %d before stage %d", input, stage_id);
        if (!ok) continue;
        commit(dev, t);
        held_since[(size_t)dev * n_inputs + input] = stage_id;
        if (input == t.out) {
          held_since[(size_t)dev * n_inputs + t.lse] = stage_id;
          if (t.dout >= 0) held_since[(size_t)dev * n_inputs + t.dout] = stage_id;
        }
      }
    }

  *n_comm = count;
  if (cross_node_load_out) std::copy(pk.cross_load.begin(), pk.cross_load.end(), cross_node_load_out);
  if (intra_node_load_out) std::copy(pk.intra_load.begin(), pk.intra_load.end(), intra_node_load_out);
  if (overflow)
    return fail(DCP_ERR_ARG, "stage_selection: transfer list of %lld entries is too small for the %lld needed",
                (long long)comm_capacity, (long long)count);
  return DCP_OK;
}
