// Launch interface between the engine (host) and the kernels.
#pragma once
#include <hip/hip_runtime.h>

#include "device_types.h"

namespace bpsx {

enum QueueCounter { kQGeo = 0 /* one per cost class */, kQGeoHead = kGeoClasses, kQReset, kQCounters };

// Work queues of one step, all in HBM, sized for every agent of a group.
struct StepQueues {
  uint32_t* counts;          // [kQCounters], see QueueCounter
  GeoQuery* queries;         // [kGeoClasses][stride]: one per moved/finished agent plus one per reset
  uint32_t stride;           // 2n
  uint32_t* reset_list;      // [n] agent indices being reset
};

struct StepParams {
  uint32_t n;          // agents in the group
  uint32_t base;       // index of the group's first agent
  uint32_t total;      // agents in the simulator (reset results live at geo[total + i])
  float max_steps;
  uint32_t reset_mode;
  uint32_t task;       // BPSX_TASK_*
  uint32_t info_width; // floats per agent in the infos output
  uint64_t seed;
  float turn_left[4], turn_right[4];  // glm::angleAxis(+-radians(10), up), x,y,z,w
  uint32_t* error_flag;
  uint64_t* counters;
  // scene rotation: per scene slot the scene-table entry its envs move to when their episode
  // ends (kNoSwap: none) and how many envs have yet to move
  uint32_t num_slots;
  const uint32_t* swap_target;
  uint32_t* swap_remaining;
  // 1: the first distance of an episode that begins in this step is measured in the next step's
  // launch (see launch_step); 0: in this one
  uint32_t defer_first_distance;
};
constexpr uint32_t kNoSwap = 0xffffffffu;

constexpr int kStepEvents = 5;  // timestamps recorded by launch_step when asked to

// One step of a group.  Q holds the step's queries, among them the first queries of the episodes
// that began in the previous step; the episodes that begin in this one are snapped on `side`
// while the searches run on `st`, and their first queries go to Qnext, the next step's queues.
// `moved` and `snapped` are events of the caller's for the fork and the join of the two streams.
void launch_step(const NavData& nav, const AgentArrays& A, const StepQueues& Q, const StepQueues& Qnext, const StepParams& P,
                 const int64_t* actions_dev, GeoSlot* slots, uint32_t geo_blocks, uint32_t snap_blocks, hipStream_t st,
                 hipStream_t side, hipEvent_t moved, hipEvent_t snapped, hipEvent_t* ev);
// Reset of a whole group, all on st; Qother (the group's other set of queues) is emptied.
void launch_reset(const NavData& nav, const AgentArrays& A, const StepQueues& Q, const StepQueues& Qother, const StepParams& P,
                  GeoSlot* slots, uint32_t geo_blocks, uint32_t snap_blocks, hipStream_t st);
void launch_snap_batch(const NavData& nav, uint32_t scene, const float* pts, uint32_t n, float* oxyz, uint32_t* oref,
                       uint32_t snap_blocks, hipStream_t st);
void launch_try_step_batch(const NavData& nav, uint32_t scene, const float* sxyz, const uint32_t* sref, const float* exyz,
                           uint32_t n, float* oxyz, uint32_t* oref, hipStream_t st);
void launch_geodesic_batch(const NavData& nav, uint32_t scene, const float* sxyz, const uint32_t* sref, const float* exyz,
                           const uint32_t* eref, uint32_t n, GeoQuery* qbuf, uint32_t* count_head /* [kGeoClasses + 1] */,
                           float* out,
                           GeoSlot* slots, uint32_t geo_blocks, uint64_t* counters, hipStream_t st);
void launch_random_points(const NavData& nav, uint32_t scene, const float* u, uint32_t n, float* oxyz, uint32_t* oref,
                          hipStream_t st);

void launch_set_swap(uint32_t* swap_target, uint32_t* swap_remaining, uint32_t slot, uint32_t target, uint32_t envs,
                     hipStream_t st);

// Wavefronts of the A* kernel that one compute unit holds at once (bounded by their LDS).
uint32_t geodesic_blocks_per_cu();

}  // namespace bpsx
