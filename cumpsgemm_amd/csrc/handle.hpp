// Library-private state behind the opaque cuMpSGEMM_handle_t.
// Plays the role of reference src/handle.hpp:7-29, src/exp_stats.hpp:7-29 and
// src/dynamic_launch.hpp:8-19, laid out for this implementation.
#pragma once
#include <hip/hip_runtime.h>
#include <cumpsgemm/cumpsgemm.h>
#include <algorithm>
#include <cstring>
#include <chrono>
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

namespace cumpsgemm_amd {

// One result slot of the exponent-statistics ring (device memory).
struct StatsSlot {
  uint32_t max_exp_bits;        // bits(max|x|) & 0x7f800000
  int32_t mode;                 // cuMpSGEMM_compute_mode_t decided for the matrix
  unsigned long long total;     // #{|x| >= ignore threshold}
  unsigned long long underflow; // #{ignore <= |x| < underflow threshold}
  uint32_t pad[2];
};
static_assert(sizeof(StatsSlot) == 32, "slot layout");

// Launch flag = compute mode (bits 0-4) + "scale B" (bit 5) + "scale A" (bit 6)
// (reference src/dynamic_launch_utils.hpp:10-41), and the flag that the
// decisions for A and B give (src/dynamic_scaling.cu:364-385): bf16x3 if
// either matrix needs it, else FP16TCEC with a scale bit per matrix that asked
// for scaling.
constexpr int kScaleABit = 0x40, kScaleBBit = 0x20, kModeMask = 0x1f;
__host__ __device__ inline int combine_launch_flag(int mode_a, int mode_b) {
  if (mode_a == CUMPSGEMM_TF32TCEC || mode_b == CUMPSGEMM_TF32TCEC) return CUMPSGEMM_TF32TCEC;
  int f = CUMPSGEMM_FP16TCEC;
  if (mode_a == CUMPSGEMM_FP16TCEC_SCALING) f |= kScaleABit;
  if (mode_b == CUMPSGEMM_FP16TCEC_SCALING) f |= kScaleBBit;
  return f;
}

// Per-workgroup partial result of a statistics pass (device scratch).
struct StatsPartial {
  uint32_t max_bits;
  uint32_t pad;
  unsigned long long total;
  unsigned long long underflow;
};

struct Profiler {
  struct Entry {
    double sum = 0.0;
    uint64_t n = 0;
  };
  bool enabled = false;
  std::unordered_map<std::string, Entry> entries;
  std::chrono::steady_clock::time_point t0;
};

constexpr unsigned kRingLength = 10000;        // reference src/exp_stats.cu:574
constexpr unsigned kMaxStatsBlocks = 4096;     // partial-result scratch entries

// Tuning knobs of the GEMM path, read from the environment once per process
// (cuMpSGEMM_reload_tuning_env() reads them again; it is meant for tests and
// experiments and must not run while another thread is inside a GEMM call).
struct Tuning {
  int packed = -1;      // CUMPSGEMM_PACKED: 0 never / 1 whenever possible take the pre-split path
  int packed_walk = -1; // CUMPSGEMM_PACKED_WALK: 0 / 1 force the one-tile / persistent pre-split kernel
  int raster_group = 0; // CUMPSGEMM_RASTER_GROUP: tile rows per column group (0: built-in choice)
  // CUMPSGEMM_EXP_FETCH_FROM_ONE_PATCH (profiler experiment, WRONG RESULTS): the
  // tile-walking pre-split kernel reads every tile's operands from one
  // L2-resident patch, which shows what its operand traffic over the fabric costs
  bool fetch_from_one_patch = false;
  int force_cls = -1;   // CUMPSGEMM_FORCE_TILE_CLASS
  int force_split = 0;  // CUMPSGEMM_FORCE_KSPLIT
  bool no_persistent = false;    // CUMPSGEMM_NO_PERSISTENT
  bool no_column_split = false;  // CUMPSGEMM_NO_COLUMN_SPLIT
  bool no_edge16_twin = false;   // CUMPSGEMM_NO_EDGE16_TWIN: never the 16x16x32 instance of the large in-loop tile
  int cut_percent = -1;          // CUMPSGEMM_CUT_PERCENT: C is cut when the model prices the two parts below this
                                 // share of the uncut plan (unset: 93, complex 96, complex bf16x3 110)
  bool no_kslices = false;       // CUMPSGEMM_NO_KSLICE_GROUPS
  bool no_fused_scaling = false; // CUMPSGEMM_NO_FUSED_SCALING
  unsigned persistent_max_steps = 32; // CUMPSGEMM_PERSISTENT_MAX_STEPS
  // CUMPSGEMM_MAX_WORKSPACE_BYTES: the pre-split path is not taken when its
  // planes would need more than this (0 keeps the path from allocating at all)
  unsigned long long max_workspace_bytes = 16ull << 30;
};
const Tuning &tuning();
} // namespace cumpsgemm_amd

struct cuMpSGEMM_handle {
  int device = 0;
  unsigned num_cus = 0;
  hipStream_t stream = nullptr;

  // ---- exponent statistics ----
  bool exp_stats_enabled = false;
  cumpsgemm_amd::StatsSlot *stats_slots = nullptr;       // [ring_length]
  cumpsgemm_amd::StatsPartial *stats_partials = nullptr; // [kMaxStatsBlocks]
  unsigned *stats_ticket = nullptr;                      // [3] self-resetting arrival counters (job 0, job 1, the pair)
  unsigned stats_ring_length = cumpsgemm_amd::kRingLength;
  unsigned stats_current_id = 1; // slots 0 / 1 are reserved presets
  float ignore_threshold = 0.0f;
  float underflow_threshold = 1.0f / 32768.0f;
  float underflow_tolerance_rate = 0.0f;

  // ---- launch-flag ring (AUTO mode) ----
  int *flag_buffer = nullptr; // [flag_ring_length]
  unsigned flag_ring_length = cumpsgemm_amd::kRingLength;
  unsigned flag_current_id = 1;
  bool flag_enabled = false;
  unsigned flag_enabled_id = 0;

  // While set, FP16TCEC GEMMs apply the power-of-two scaling of these
  // statistics slots / this launch flag inside the kernel (the mode pipelines
  // switch it on around their GEMM when A and B are to be left untouched).
  bool fused_scaling = false;
  unsigned fused_slot_a = 0, fused_slot_b = 0, fused_flag = 0;

  // workspace of the pre-split (packed) GEMM path: grows on demand, freed with
  // the handle
  void *pack_ws = nullptr;
  unsigned long long pack_ws_bytes = 0;
  // A HIP graph captured while the pre-split path ran holds the address of
  // pack_ws: from then on that buffer is never freed before the handle is
  // destroyed (a later, larger call gets a new one and the old one is parked
  // here), so replays of the graph keep reading and writing memory they own.
  bool pack_ws_captured = false;
  std::vector<void *> retired_ws;
  // Set for the duration of one call by the entry point that allocates
  // nothing: the planes go to this caller-independent buffer (a static device
  // array), the pre-split path is taken whatever the shape rules say, and no
  // allocation, free or synchronisation happens.
  void *ws_override = nullptr;
  unsigned long long ws_override_bytes = 0;

  // The rings, partials and workspaces above are shared by every call on the
  // handle, so work of the handle on two streams must not overlap: when the
  // stream changes, the new one is made to wait (on the device, through this
  // event) for what was queued on the old one.
  hipEvent_t order_event = nullptr;

  // pinned host word for small read-backs
  unsigned long long *host_scratch = nullptr; // [4]

  cumpsgemm_amd::Profiler profiler;
};

namespace cumpsgemm_amd {
// Wall-clock bracket around a launch when profiling is on (reference:
// cutf profiler start_timer_sync / stop_timer_sync, src/cumpsgemm.cu:263-271).
struct ProfileScope {
  cuMpSGEMM_handle *h;
  const char *name;
  ProfileScope(cuMpSGEMM_handle *handle, const char *label);
  ~ProfileScope();
};

void check_hip(hipError_t err, const char *what);

// Statistics of the two operands of a GEMM with one launch per pass instead
// of two; same results and slot numbering as exp_stats_ext / exp_max_ext
// called for A, then for B.
template <class T> struct MatrixView {
  const T *ptr;
  unsigned m, n, ld, batch, stride;
};
// flag_id >= 0: the second pass also writes launch flag flag_id from the two
// decisions (what set_dynamic_launch_buffer_by_exp_stats would do in a launch
// of its own).
template <class T>
void exp_stats_pair(cuMpSGEMM_handle *h, const MatrixView<T> &a, const MatrixView<T> &b, unsigned &a_id,
                    unsigned &b_id, int flag_id = -1);
template <class T>
void exp_max_pair(cuMpSGEMM_handle *h, const MatrixView<T> &a, const MatrixView<T> &b, unsigned &a_id,
                  unsigned &b_id);
} // namespace cumpsgemm_amd
