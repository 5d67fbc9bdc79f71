// Host side of libbpsx: the C ABI declared in include/bpsx.h, device memory ownership and
// kernel sequencing.  The counterpart of RolloutGenerator / EnvironmentGroup
// (simulator.cpp:1180-1330, 1332-1700) without worker threads: a step is a short chain of
// kernels on the caller's HIP stream.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "../../include/bpsx.h"
#include "errors.h"
#include "kernels.h"
#include "navmesh_host.h"

using namespace bpsx;

#define HIP_TRY(expr)                                                                            \
  do {                                                                                           \
    hipError_t e_ = (expr);                                                                      \
    if (e_ != hipSuccess) return fail(BPSX_E_HIP, std::string(#expr) + ": " + hipGetErrorString(e_)); \
  } while (0)

namespace {

const char* const kKernelNames[BPSX_NUM_KERNELS] = {"step_move", "reset_snap", "geodesic", "step_finish"};

struct Group {
  // Two sets of queues, used in turn: a step's launch serves Q[turn] and puts the first queries
  // of the episodes that begin in it into the other set, which the next step serves.
  StepQueues Q[2] = {};
  int turn = 0;
  hipEvent_t moved = nullptr, snapped = nullptr;   // fork and join of the side stream within a step
  int64_t* d_actions = nullptr;
  int64_t* h_actions = nullptr;  // pinned staging for host-side action arrays
  hipEvent_t ev[kStepEvents] = {};
  bool in_flight = false;
  bool profiled = false;
  int record = -1;               // ring entry of the step in flight
};

// A step that has been enqueued and whose completion the host has not yet seen.  The host may
// run ahead of the device by kStepRing steps (stream-ordered stepping, bpsx_set_stream_ordered):
// what a step brings back for the host (how many envs of each scene slot are still on a scene
// that is leaving) lands in the step's own pinned buffer and is looked at when its event is
// found complete.
constexpr int kStepRing = 4;
struct StepRecord {
  hipEvent_t done = nullptr;
  uint32_t* remaining = nullptr;   // pinned, one word per scene slot
  uint64_t ordinal = 0;            // sim->steps_started when the step was enqueued
  bool has_remaining = false;
};

template <class T>
int dev_alloc(T** p, size_t count) {
  HIP_TRY(hipMalloc((void**)p, std::max<size_t>(count, 1) * sizeof(T)));
  HIP_TRY(hipMemset(*p, 0, std::max<size_t>(count, 1) * sizeof(T)));
  return BPSX_OK;
}

}  // namespace

// ---- scratch of the allocation-free geodesic entry point (bpsx_geodesic_static).  One array per
// GPU, held until the process ends: the queries built from the caller's arrays, the queue
// counters, and the node pools of the kStaticBlocks * 2 wavefronts that serve the queue.
namespace {
constexpr uint32_t kStaticBlocks = 16;
constexpr size_t kStaticQueriesBytes = (size_t)BPSX_STATIC_MAX_QUERIES * sizeof(GeoQuery);
constexpr size_t kStaticCountsBytes = 512;
static_assert((kGeoClasses + 2) * sizeof(uint32_t) <= kStaticCountsBytes, "queue counters must fit their part");
static_assert(kStaticQueriesBytes % 256 == 0 && sizeof(GeoSlot) % 256 == 0, "parts of the scratch stay aligned");
constexpr size_t kStaticSlotsBytes = (size_t)kStaticBlocks * 2 * sizeof(GeoSlot);
constexpr size_t kStaticBytes = kStaticQueriesBytes + kStaticCountsBytes + kStaticSlotsBytes;
constexpr int kMaxDevices = 64;
unsigned char* g_static_scratch[kMaxDevices] = {};   // device address of `scratch` on each GPU that has been set up
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticBytes];

// Looks the array's address up on the current device, once per device.
static int static_scratch_setup(int device) {
  if (device < 0 || device >= kMaxDevices) return fail(BPSX_E_UNSUPPORTED, "device ordinal beyond the table of static scratch arrays");
  if (g_static_scratch[device]) return BPSX_OK;
  unsigned char* ptr = nullptr;
  HIP_TRY(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
  if (!ptr) return fail(BPSX_E_HIP, "hipGetSymbolAddress returned a null address for the static scratch array");
  g_static_scratch[device] = ptr;
  return BPSX_OK;
}

// First-fit allocator over one of the concatenated navmesh arrays (units = elements).  Scenes
// come and go with scene rotation; neighbouring free ranges are merged on release.
struct Arena {
  size_t cap = 0;
  std::vector<std::pair<size_t, size_t>> free_ranges;   // (offset, length), sorted by offset
  void init(size_t capacity) { cap = capacity; free_ranges.assign(1, {0, capacity}); }
  bool take(size_t len, size_t* off) {
    if (len == 0) { *off = 0; return true; }
    for (size_t i = 0; i < free_ranges.size(); ++i) {
      if (free_ranges[i].second < len) continue;
      *off = free_ranges[i].first;
      free_ranges[i].first += len;
      free_ranges[i].second -= len;
      if (!free_ranges[i].second) free_ranges.erase(free_ranges.begin() + (long)i);
      return true;
    }
    return false;
  }
  void give(size_t off, size_t len) {
    if (!len) return;
    size_t i = 0;
    while (i < free_ranges.size() && free_ranges[i].first < off) ++i;
    free_ranges.insert(free_ranges.begin() + (long)i, {off, len});
    for (size_t k = 0; k + 1 < free_ranges.size();) {
      if (free_ranges[k].first + free_ranges[k].second == free_ranges[k + 1].first) {
        free_ranges[k].second += free_ranges[k + 1].second;
        free_ranges.erase(free_ranges.begin() + (long)k + 1);
      } else {
        ++k;
      }
    }
  }
};
// Where one resident scene lives in the arrays.
struct SceneRanges {
  size_t poly = 0, npoly = 0, bv = 0, nbv = 0, tri = 0, ntri = 0, dv = 0, ndv = 0, ep = 0, nep = 0;
  bool used = false;
};
// A scene slot has two scene-table entries (slot and slot + num_active_scenes): the scene its
// envs are on and, during a swap, the scene they are moving to.
struct SceneSlot {
  uint32_t current = 0;         // scene-table entry of the resident scene
  uint32_t target = kNoSwap;    // entry of the scene being moved to, if a swap is in progress or just done
  uint64_t target_ordinal = 0;  // the step that made it the target: earlier steps' counts say nothing about this swap
  // automatic rotation (SceneSwapper, simulator.cpp:1063-1154)
  uint32_t active_scene = 0;    // dataset index of the scene the slot's envs are on or are moving to
  uint32_t load_entry = kNoSwap;          // scene-table entry the loader thread is filling / has filled
  std::atomic<uint32_t> load_state{0};    // 0 none, 1 requested, 2 resident and ready, 3 failed
  // A slot's two scene-table entries are never touched by both threads at once: the loader
  // thread writes load_entry's ranges and table entry only between load_state 1 and 2 or 3, the
  // stepping thread reads or releases them only outside that interval.
};
// One scene of the dataset as handed to bpsx_add_scene: kept as bytes while it is not resident.
struct PoolScene {
  std::vector<uint8_t> blob;
  std::vector<float> episodes;
  std::unique_ptr<HostScene> parsed;   // until finalize
};

// ---- counter-based stream of the scene choices (same integer arithmetic as the kernels' reset stream)
static uint64_t mix64_host(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
static uint32_t scene_draw(uint64_t seed, uint64_t k) {
  const uint64_t key = mix64_host(seed + 0x9E3779B97F4A7C15ull * 0x100000000ull + 0xD1B54A32D192ED03ull);
  return (uint32_t)(mix64_host(key + 0x9E3779B97F4A7C15ull * (k + 1)) >> 32);
}

struct bpsx_sim {
  bpsx_config cfg{};
  bool finalized = false;
  uint32_t num_groups = 1, envs_per_group = 0;
  // navmesh arrays
  PolyRec* d_polys = nullptr;
  AEdge* d_aedges = nullptr;
  BVNodeDev* d_bv = nullptr;
  uint8_t* d_dtris = nullptr;
  float* d_dverts = nullptr;
  SceneDev* d_scenes = nullptr;
  float* d_episodes = nullptr;
  NavData nav{};
  Arena ar_poly, ar_bv, ar_tri, ar_dv, ar_ep;
  bool fixed_regions = false;        // automatic rotation: one region per scene-table entry instead of the arenas
  SceneRanges region;                // n*: elements of one region in each array
  std::vector<SceneRanges> ranges;   // per scene-table entry
  std::unique_ptr<SceneSlot[]> slots;
  // dataset and automatic rotation
  std::vector<PoolScene> pool;           // every scene added, in call order
  std::vector<uint32_t> inactive;        // dataset indices not resident (simulator.cpp:1518-1534)
  uint64_t scene_draws = 0;              // draws taken from the scene-choice stream
  bool rotating = false;
  std::mutex arena_mu;                   // the arenas are used by the loader thread too
  std::thread loader;
  std::mutex loader_mu;
  std::condition_variable loader_cv;
  std::deque<uint32_t> loader_requests;  // slots waiting for their next scene
  bool loader_exit = false;
  std::string loader_error;              // first failure of the loader thread (guarded by loader_mu)
  bool loader_error_reported = false;    // step_end has returned it once
  hipStream_t upload_stream = nullptr;   // uploads of scenes that come in while the simulation runs
  hipStream_t side = nullptr;            // a step's snaps of new episodes, next to its searches (default priority)
  uint32_t* h_swap_remaining = nullptr;  // d_swap_remaining as of the newest step whose completion has been seen
  StepRecord ring[kStepRing];
  int ring_head = 0, ring_count = 0;     // oldest outstanding record, number outstanding
  bool stream_ordered = false;           // step_end leaves the waiting to the stream (bpsx_set_stream_ordered)
  std::vector<uint32_t> rotation_log;    // (step ordinal, slot, dataset index) of swaps made available
  uint64_t steps_started = 0, env_steps_taken = 0;
  uint32_t* d_swap_target = nullptr;
  uint32_t* d_swap_remaining = nullptr;
  uint64_t swaps_completed = 0;
  AgentArrays A{};
  std::vector<void*> owned;  // every device allocation, for destroy
  std::vector<Group> groups;
  GeoSlot* d_slots = nullptr;
  uint32_t geo_blocks = 0, snap_blocks = 0;
  uint32_t* d_error = nullptr;
  uint64_t* d_counters = nullptr;
  float turn_left[4], turn_right[4];
  // profiling
  bool profiling = false;
  double kernel_ms[BPSX_NUM_KERNELS] = {};
  uint64_t profiled_steps = 0;
  // scratch for the batched query entry points
  void* d_batch = nullptr;
  size_t batch_bytes = 0;
  uint32_t* d_batch_counts = nullptr;

  template <class T>
  int alloc(T** p, size_t count) {
    const int rc = dev_alloc(p, count);
    if (rc == BPSX_OK) owned.push_back((void*)*p);
    return rc;
  }
  uint32_t info_width() const { return cfg.task == BPSX_TASK_POINTNAV ? 3u : 1u; }
  StepParams params(uint32_t group) const {
    StepParams P{};
    P.n = envs_per_group;
    P.base = group * envs_per_group;
    P.total = cfg.num_environments;
    P.max_steps = (float)(cfg.max_steps ? cfg.max_steps : BPSX_MAX_STEPS);
    P.reset_mode = cfg.reset_mode;
    P.task = cfg.task;
    P.info_width = info_width();
    P.seed = cfg.seed;
    memcpy(P.turn_left, turn_left, 16);
    memcpy(P.turn_right, turn_right, 16);
    P.error_flag = d_error;
    P.counters = d_counters;
    P.num_slots = cfg.num_active_scenes;
    P.swap_target = d_swap_target;
    P.swap_remaining = d_swap_remaining;
    return P;
  }
};

extern "C" {

int bpsx_create(const bpsx_config* cfg, bpsx_sim** out) {
  if (!cfg || !out) return fail(BPSX_E_INVAL, "create: null argument");
  if (!cfg->num_environments || !cfg->num_active_scenes) return fail(BPSX_E_INVAL, "create: zero environments or scenes");
  const uint32_t groups = cfg->double_buffered ? 2 : 1;
  if (cfg->num_environments % cfg->num_active_scenes != 0)
    return fail(BPSX_E_INVAL, "create: num_environments is not a multiple of num_active_scenes");
  if (cfg->num_active_scenes % groups != 0)
    return fail(BPSX_E_INVAL, "create: num_active_scenes is not a multiple of the number of groups");
  if (cfg->reset_mode > BPSX_RESET_SAMPLED) return fail(BPSX_E_INVAL, "create: unknown reset_mode");
  if (cfg->task > BPSX_TASK_EXPLORATION) return fail(BPSX_E_INVAL, "create: unknown task");
  if (cfg->task == BPSX_TASK_EXPLORATION && cfg->max_steps > 8192)
    return fail(BPSX_E_UNSUPPORTED, "create: the exploration task keeps one cell per step, max_steps <= 8192");
  int ndev = 0;
  HIP_TRY(hipGetDeviceCount(&ndev));
  if (cfg->gpu_id < 0 || cfg->gpu_id >= ndev) return fail(BPSX_E_INVAL, "create: gpu_id out of range");
  bpsx_sim* s = new bpsx_sim();
  s->cfg = *cfg;
  s->num_groups = groups;
  s->envs_per_group = cfg->num_environments / groups;
  // glm::angleAxis(+-glm::radians(10.f), (0,1,0)) evaluated with the host libm, as the
  // reference's static initialisers do (simulator.cpp:52-60)
  const float a = BPSX_TURN_DEGREES * 0.01745329251994329576923690768489f;
  s->turn_left[0] = 0; s->turn_left[1] = sinf(a * 0.5f); s->turn_left[2] = 0; s->turn_left[3] = cosf(a * 0.5f);
  s->turn_right[0] = 0; s->turn_right[1] = sinf(-a * 0.5f); s->turn_right[2] = 0; s->turn_right[3] = cosf(-a * 0.5f);
  *out = s;
  return BPSX_OK;
}

int bpsx_add_scene(bpsx_sim* sim, const void* navmesh_bytes, size_t navmesh_size, const float* episodes,
                   uint32_t num_episodes) {
  if (!sim || !navmesh_bytes) return fail(BPSX_E_INVAL, "add_scene: null argument");
  if (sim->finalized) return fail(BPSX_E_STATE, "add_scene: simulator already finalized");
  if (sim->cfg.reset_mode == BPSX_RESET_EPISODES && (!episodes || !num_episodes))
    return fail(BPSX_E_INVAL, "add_scene: episode-table reset needs at least one episode");
  PoolScene ps;
  ps.parsed.reset(new HostScene());
  const int rc = parse_navmesh((const uint8_t*)navmesh_bytes, navmesh_size, ps.parsed.get());
  if (rc) return rc;
  if (episodes && num_episodes) ps.episodes.assign(episodes, episodes + (size_t)num_episodes * 10);
  ps.parsed->episodes = ps.episodes;
  ps.parsed->dev.ep_count = num_episodes;
  ps.blob.assign((const uint8_t*)navmesh_bytes, (const uint8_t*)navmesh_bytes + navmesh_size);
  sim->pool.push_back(std::move(ps));
  return BPSX_OK;
}

// Places one parsed scene into the arrays and writes its scene-table entry.
// The copies go out on `st` and have completed when the function returns; other streams are
// not waited for.
static int upload_scene(bpsx_sim* sim, HostScene& s, uint32_t entry, hipStream_t st) {
  SceneRanges r;
  r.npoly = s.polys.size(); r.nbv = s.bv.size(); r.ntri = s.dtris.size() / 4; r.ndv = s.dverts.size() / 3;
  r.nep = s.episodes.size() / 10;
  if (sim->fixed_regions) {
    // automatic rotation: every scene-table entry owns a region that holds the largest scene of
    // the pool, so a load can neither fail nor depend on what came and went before it
    const SceneRanges& m = sim->region;
    if (r.npoly > m.npoly || r.nbv > m.nbv || r.ntri > m.ntri || r.ndv > m.ndv || r.nep > m.nep)
      return fail(BPSX_E_UNSUPPORTED, "scene is larger than the largest scene the simulator was finalized with");
    r.poly = entry * m.npoly; r.bv = entry * m.nbv; r.tri = entry * m.ntri; r.dv = entry * m.ndv; r.ep = entry * m.nep;
    r.used = true;
    std::lock_guard<std::mutex> lk(sim->arena_mu);
    sim->ranges[entry] = r;
  } else {
    std::lock_guard<std::mutex> lk(sim->arena_mu);
    const bool a = sim->ar_poly.take(r.npoly, &r.poly);
    const bool b = a && sim->ar_bv.take(r.nbv, &r.bv);
    const bool c = b && sim->ar_tri.take(r.ntri, &r.tri);
    const bool d = c && sim->ar_dv.take(r.ndv, &r.dv);
    const bool e = d && sim->ar_ep.take(r.nep, &r.ep);
    if (!e) {
      if (a) sim->ar_poly.give(r.poly, r.npoly);
      if (b) sim->ar_bv.give(r.bv, r.nbv);
      if (c) sim->ar_tri.give(r.tri, r.ntri);
      if (d) sim->ar_dv.give(r.dv, r.ndv);
      return fail(BPSX_E_UNSUPPORTED, "scene does not fit the space reserved for scene rotation");
    }
    r.used = true;
    sim->ranges[entry] = r;
  }
  s.dev.poly_base = (uint32_t)r.poly; s.dev.bv_base = (uint32_t)r.bv; s.dev.ep_base = (uint32_t)r.ep;
  s.dev.ep_count = (uint32_t)r.nep;
  for (auto& p : s.polys) { p.tri_base += (uint32_t)r.tri; p.dvert_base += (uint32_t)r.dv; }
  const auto H2D = hipMemcpyHostToDevice;
  HIP_TRY(hipMemcpyAsync(sim->d_polys + r.poly, s.polys.data(), r.npoly * sizeof(PolyRec), H2D, st));
  HIP_TRY(hipMemcpyAsync(sim->d_aedges + r.poly * kEdgeStride, s.aedges.data(), s.aedges.size() * sizeof(AEdge), H2D, st));
  if (r.nbv) HIP_TRY(hipMemcpyAsync(sim->d_bv + r.bv, s.bv.data(), r.nbv * sizeof(BVNodeDev), H2D, st));
  if (r.ntri) HIP_TRY(hipMemcpyAsync(sim->d_dtris + r.tri * 4, s.dtris.data(), s.dtris.size(), H2D, st));
  if (r.ndv) HIP_TRY(hipMemcpyAsync(sim->d_dverts + r.dv * 3, s.dverts.data(), s.dverts.size() * 4, H2D, st));
  if (r.nep) HIP_TRY(hipMemcpyAsync(sim->d_episodes + r.ep * 10, s.episodes.data(), s.episodes.size() * 4, H2D, st));
  HIP_TRY(hipMemcpyAsync(sim->d_scenes + entry, &s.dev, sizeof(SceneDev), H2D, st));
  HIP_TRY(hipStreamSynchronize(st));
  return BPSX_OK;
}
static void release_scene(bpsx_sim* sim, uint32_t entry) {
  std::lock_guard<std::mutex> lk(sim->arena_mu);
  SceneRanges& r = sim->ranges[entry];
  if (!r.used) return;
  if (sim->fixed_regions) { r = SceneRanges{}; return; }
  sim->ar_poly.give(r.poly, r.npoly); sim->ar_bv.give(r.bv, r.nbv); sim->ar_tri.give(r.tri, r.ntri);
  sim->ar_dv.give(r.dv, r.ndv); sim->ar_ep.give(r.ep, r.nep);
  r = SceneRanges{};
}

// ---- automatic scene rotation.  Counterpart of SceneSwapper + BackgroundSceneLoader
// (simulator.cpp:361-551, 1063-1154): a loader thread parses the next scene of a slot and
// uploads it on a stream of its own while the simulation steps; step_start makes a scene that
// has become resident the slot's target (preStep), the envs move over when their episodes end,
// and step_end, once none is left on the old scene, frees it and draws the slot's next scene
// from the scenes that are not resident (postStep / startSceneSwap).
static void loader_loop(bpsx_sim* sim) {
  (void)hipSetDevice(sim->cfg.gpu_id);
  auto last = std::chrono::steady_clock::now() - std::chrono::hours(1);
  for (;;) {
    uint32_t slot;
    {
      std::unique_lock<std::mutex> lk(sim->loader_mu);
      sim->loader_cv.wait(lk, [&] { return sim->loader_exit || !sim->loader_requests.empty(); });
      if (sim->loader_exit) return;
      slot = sim->loader_requests.front();
      sim->loader_requests.pop_front();
    }
    // at most one load per interval (the reference's RATE_LIMIT of one second, simulator.cpp:545-548)
    const auto gap = std::chrono::milliseconds(sim->cfg.rotation_interval_ms);
    const auto now = std::chrono::steady_clock::now();
    if (now - last < gap) {
      std::unique_lock<std::mutex> lk(sim->loader_mu);
      sim->loader_cv.wait_for(lk, gap - (now - last), [&] { return sim->loader_exit; });
      if (sim->loader_exit) return;
    }
    last = std::chrono::steady_clock::now();
    SceneSlot& sl = sim->slots[slot];
    const PoolScene& ps = sim->pool[sl.active_scene];
    HostScene hs;
    int rc = parse_navmesh(ps.blob.data(), ps.blob.size(), &hs);
    if (!rc) {
      hs.episodes = ps.episodes;
      rc = upload_scene(sim, hs, sl.load_entry, sim->upload_stream);
    }
    if (rc) {
      // step_end reports it; the slot keeps its scene and stops rotating
      std::lock_guard<std::mutex> lk(sim->loader_mu);
      if (sim->loader_error.empty())
        sim->loader_error = "scene " + std::to_string(sl.active_scene) + " for slot " + std::to_string(slot) + ": " + last_error_message();
      sl.load_state.store(3, std::memory_order_release);
    } else {
      sl.load_state.store(2, std::memory_order_release);
    }
  }
}
// SceneSwapper::startSceneSwap (simulator.cpp:1093-1106): a scene that is not resident, drawn
// uniformly, changes places with the slot's scene and is sent to the loader.
static void start_scene_swap(bpsx_sim* sim, uint32_t slot) {
  if (sim->inactive.empty()) return;
  SceneSlot& sl = sim->slots[slot];
  const uint32_t r = scene_draw(sim->cfg.seed, sim->scene_draws++);
  const uint32_t pos = (uint32_t)(((uint64_t)r * (uint64_t)sim->inactive.size()) >> 32);
  std::swap(sim->inactive[pos], sl.active_scene);
  const uint32_t S = sim->cfg.num_active_scenes;
  sl.load_entry = sl.current < S ? slot + S : slot;   // the slot's other scene-table entry
  sl.load_state.store(1, std::memory_order_release);
  {
    std::lock_guard<std::mutex> lk(sim->loader_mu);
    sim->loader_requests.push_back(slot);
  }
  sim->loader_cv.notify_one();
}
// SceneSwapper::preStep: scenes that have become resident are what their slots' envs move to
// from this step on.  The switch is made by a kernel on the step's stream, in order with the step.
static int rotation_pre_step(bpsx_sim* sim, hipStream_t st) {
  const uint32_t S = sim->cfg.num_active_scenes, per = sim->cfg.num_environments / S;
  for (uint32_t slot = 0; slot < S; ++slot) {
    SceneSlot& sl = sim->slots[slot];
    if (sl.load_state.load(std::memory_order_acquire) != 2) continue;
    sl.load_state.store(0, std::memory_order_relaxed);
    sl.target = sl.load_entry;
    sl.target_ordinal = sim->steps_started;
    launch_set_swap(sim->d_swap_target, sim->d_swap_remaining, slot, sl.target, per, st);
    HIP_TRY(hipGetLastError());
    sim->h_swap_remaining[slot] = per;
    sim->rotation_log.push_back((uint32_t)sim->steps_started);
    sim->rotation_log.push_back(slot);
    sim->rotation_log.push_back(sl.active_scene);
  }
  return BPSX_OK;
}
// SceneSwapper::postStep: a slot whose envs have all moved gives its old scene's space back and
// starts loading its next scene.  `rec` is a step that has completed: its counts are what the
// device held after it.  Steps enqueued after it do not read the old scene either (every env of
// the slot had left it), so its space can go to the loader at once.
static void rotation_post_step(bpsx_sim* sim, const StepRecord& rec) {
  const uint32_t S = sim->cfg.num_active_scenes;
  for (uint32_t slot = 0; slot < S; ++slot) {
    SceneSlot& sl = sim->slots[slot];
    if (sl.target == kNoSwap || sl.target == sl.current || sl.target_ordinal > rec.ordinal) continue;
    sim->h_swap_remaining[slot] = rec.remaining[slot];
    if (rec.remaining[slot] != 0) continue;
    release_scene(sim, sl.current);
    sl.current = sl.target;   // the device keeps the target: envs already on it ignore it
    sim->swaps_completed++;
    if (sim->rotating) start_scene_swap(sim, slot);
  }
}

// Takes the records whose steps have completed off the ring, oldest first.  wait_for: number of
// records that must leave, waiting for their events if need be (ring_count: all of them).
static int retire_steps(bpsx_sim* sim, int wait_for) {
  while (sim->ring_count > 0) {
    StepRecord& rec = sim->ring[sim->ring_head];
    if (wait_for > 0) {
      HIP_TRY(hipEventSynchronize(rec.done));
    } else {
      const hipError_t q = hipEventQuery(rec.done);
      if (q == hipErrorNotReady) break;
      if (q != hipSuccess) return fail(BPSX_E_HIP, std::string("hipEventQuery: ") + hipGetErrorString(q));
    }
    if (rec.has_remaining && sim->rotating) rotation_post_step(sim, rec);
    sim->ring_head = (sim->ring_head + 1) % kStepRing;
    sim->ring_count--;
    wait_for--;
  }
  return BPSX_OK;
}
// Everything enqueued by earlier steps has completed when this returns.
static int quiesce(bpsx_sim* sim) { return retire_steps(sim, sim->ring_count); }

int bpsx_finalize(bpsx_sim* sim) {
  if (!sim) return fail(BPSX_E_INVAL, "finalize: null simulator");
  if (sim->finalized) return fail(BPSX_E_STATE, "finalize: called twice");
  const uint32_t S = sim->cfg.num_active_scenes;
  if (sim->pool.size() < S) return fail(BPSX_E_INVAL, "finalize: fewer scenes added than num_active_scenes");
  HIP_TRY(hipSetDevice(sim->cfg.gpu_id));
  // ---- which scenes of the dataset start resident: selection sampling over the dataset in
  // order, like simulator.cpp:1518-1534 (there on the generator's mt19937, here on the
  // counter-based stream): scene i is taken when u * (D - i) < scenes still to take.  With as
  // many scenes as slots every scene is taken, in order.
  {
    const uint32_t D = (uint32_t)sim->pool.size();
    std::vector<uint32_t> active;
    uint32_t i = 0;
    for (; i < D && active.size() < S; ++i) {
      const float weight = (float)(scene_draw(sim->cfg.seed, sim->scene_draws++) >> 8) * (1.0f / 16777216.0f);
      if (weight * (float)(D - i) < (float)(S - (uint32_t)active.size())) active.push_back(i);
      else sim->inactive.push_back(i);
    }
    for (; i < D; ++i) sim->inactive.push_back(i);
    sim->slots.reset(new SceneSlot[S]);
    for (uint32_t k = 0; k < S; ++k) sim->slots[k].active_scene = active[k];
  }
  // ---- navmesh arrays: every scene is a range of each array.
  // Without automatic rotation the scenes lie one after the other, with room for scenes that the
  // caller may swap in (bpsx_swap_scene; their sizes are not known: scene_reserve times the
  // initial scenes plus the largest one, handed out first-fit).  With automatic rotation any
  // scene of the pool may become resident, two per slot while a swap is in progress, in any
  // order: each of the 2 S scene-table entries owns a region as large as the largest scene of
  // the pool, so that no sequence of swaps can fail for lack of a free range of the right size
  // (S = 128 mazes of 32k polygons: 2.4 GB of the GPU's 288).
  const bool will_rotate = sim->cfg.rotate_scenes && !sim->inactive.empty();
  const double k = sim->cfg.scene_reserve > 0 ? (double)sim->cfg.scene_reserve : 3.0;
  if (k < 1.0) return fail(BPSX_E_INVAL, "finalize: scene_reserve must be at least 1");
  auto capacity = [&](auto size_of, size_t* region) {
    size_t total = 0, largest = 0;
    for (uint32_t i = 0; i < S; ++i) total += size_of(*sim->pool[sim->slots[i].active_scene].parsed);
    for (auto& ps : sim->pool) largest = std::max(largest, (size_t)size_of(*ps.parsed));
    *region = largest;
    return will_rotate ? 2 * (size_t)S * largest + 64 : (size_t)((double)total * k) + largest + 64;
  };
  sim->fixed_regions = will_rotate;
  const size_t cpoly = capacity([](const HostScene& s) { return s.polys.size(); }, &sim->region.npoly);
  const size_t cbv = capacity([](const HostScene& s) { return s.bv.size(); }, &sim->region.nbv);
  const size_t ctri = capacity([](const HostScene& s) { return s.dtris.size() / 4; }, &sim->region.ntri);
  const size_t cdv = capacity([](const HostScene& s) { return s.dverts.size() / 3; }, &sim->region.ndv);
  const size_t cep = capacity([](const HostScene& s) { return s.episodes.size() / 10; }, &sim->region.nep);
  if (cpoly > 0xfffffff0ull || ctri > 0xfffffff0ull) return fail(BPSX_E_UNSUPPORTED, "finalize: navmeshes too large");
  int rc;
  if ((rc = sim->alloc(&sim->d_polys, cpoly))) return rc;
  if ((rc = sim->alloc(&sim->d_aedges, cpoly * kEdgeStride))) return rc;
  if ((rc = sim->alloc(&sim->d_bv, cbv))) return rc;
  if ((rc = sim->alloc(&sim->d_dtris, ctri * 4))) return rc;
  if ((rc = sim->alloc(&sim->d_dverts, cdv * 3))) return rc;
  if ((rc = sim->alloc(&sim->d_scenes, 2 * (size_t)S))) return rc;
  if ((rc = sim->alloc(&sim->d_episodes, cep * 10))) return rc;
  if ((rc = sim->alloc(&sim->d_swap_target, S)) || (rc = sim->alloc(&sim->d_swap_remaining, S))) return rc;
  sim->ar_poly.init(cpoly); sim->ar_bv.init(cbv); sim->ar_tri.init(ctri); sim->ar_dv.init(cdv); sim->ar_ep.init(cep);
  sim->ranges.assign(2 * (size_t)S, SceneRanges{});
  sim->nav = NavData{sim->d_polys, sim->d_aedges, sim->d_bv, sim->d_dtris, sim->d_dverts, sim->d_scenes, sim->d_episodes};
  {
    std::vector<uint32_t> none(S, kNoSwap);
    HIP_TRY(hipMemcpy(sim->d_swap_target, none.data(), (size_t)S * 4, hipMemcpyHostToDevice));
  }
  HIP_TRY(hipStreamCreateWithFlags(&sim->upload_stream, hipStreamNonBlocking));
  HIP_TRY(hipStreamCreateWithFlags(&sim->side, hipStreamNonBlocking));
  HIP_TRY(hipHostMalloc((void**)&sim->h_swap_remaining, (size_t)S * 4, hipHostMallocDefault));
  memset(sim->h_swap_remaining, 0, (size_t)S * 4);
  for (StepRecord& rec : sim->ring) {
    HIP_TRY(hipEventCreateWithFlags(&rec.done, hipEventDisableTiming));
    HIP_TRY(hipHostMalloc((void**)&rec.remaining, (size_t)S * 4, hipHostMallocDefault));
    memset(rec.remaining, 0, (size_t)S * 4);
  }
  for (uint32_t i = 0; i < S; ++i) {
    sim->slots[i].current = i;
    if ((rc = upload_scene(sim, *sim->pool[sim->slots[i].active_scene].parsed, i, sim->upload_stream))) return rc;
  }
  // the parsed copies are not needed any more; the bytes stay only if scenes will rotate
  sim->rotating = will_rotate;
  for (auto& ps : sim->pool) {
    ps.parsed.reset();
    if (!sim->rotating) { ps.blob.clear(); ps.blob.shrink_to_fit(); ps.episodes.clear(); ps.episodes.shrink_to_fit(); }
  }

  // ---- agent state
  const size_t N = sim->cfg.num_environments;
  AgentArrays& A = sim->A;
  if ((rc = sim->alloc(&A.pos, N * 3)) || (rc = sim->alloc(&A.rot, N * 4)) || (rc = sim->alloc(&A.goal, N * 3)) ||
      (rc = sim->alloc(&A.nav_xyz, N * 3)) || (rc = sim->alloc(&A.nav_ref, N)) || (rc = sim->alloc(&A.goal_xyz, N * 3)) ||
      (rc = sim->alloc(&A.goal_ref, N)) || (rc = sim->alloc(&A.prev_pos, N * 3)) || (rc = sim->alloc(&A.info_prev, N)) ||
      (rc = sim->alloc(&A.cum, N)) || (rc = sim->alloc(&A.init, N)) || (rc = sim->alloc(&A.rew_prev, N)) ||
      (rc = sim->alloc(&A.step, N)) || (rc = sim->alloc(&A.scene, N)) || (rc = sim->alloc(&A.episode, N)) ||
      (rc = sim->alloc(&A.nresets, N)) || (rc = sim->alloc(&A.flags, N)) || (rc = sim->alloc(&A.dist_ok, N)) || (rc = sim->alloc(&A.last_cost, N)) || (rc = sim->alloc(&A.geo, 2 * N)) ||
      (rc = sim->alloc(&A.rewards, N)) || (rc = sim->alloc(&A.masks, N)) || (rc = sim->alloc(&A.infos, N * sim->info_width())) ||
      (rc = sim->alloc(&A.polars, N * 2)))
    return rc;
  if (sim->cfg.task == BPSX_TASK_EXPLORATION) {
    A.cell_cap = sim->cfg.max_steps ? sim->cfg.max_steps : BPSX_MAX_STEPS;
    if ((rc = sim->alloc(&A.exp_init, N * 3)) || (rc = sim->alloc(&A.exp_inv, N * 4)) ||
        (rc = sim->alloc(&A.exp_cells, N * (size_t)A.cell_cap * 3)) || (rc = sim->alloc(&A.exp_count, N)))
      return rc;
  }
  {
    // env -> scene: contiguous blocks of N / scenes (simulator.cpp:1205-1221, 1578-1592)
    std::vector<uint32_t> scene(N);
    const size_t per = N / sim->cfg.num_active_scenes;
    for (size_t i = 0; i < N; ++i) scene[i] = (uint32_t)(i / per);
    HIP_TRY(hipMemcpy(A.scene, scene.data(), N * 4, hipMemcpyHostToDevice));
    std::vector<float> rot(N * 4, 0.f);
    for (size_t i = 0; i < N; ++i) rot[i * 4 + 3] = 1.f;
    HIP_TRY(hipMemcpy(A.rot, rot.data(), N * 16, hipMemcpyHostToDevice));
  }
  if ((rc = sim->alloc(&sim->d_error, 1)) || (rc = sim->alloc(&sim->d_counters, BPSX_NUM_COUNTERS))) return rc;
  if ((rc = sim->alloc(&sim->d_batch_counts, kGeoClasses + 2))) return rc;

  // ---- A* wavefronts: as many as the LDS of the device holds at once, not one per agent
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, sim->cfg.gpu_id));
  uint32_t per_cu = geodesic_blocks_per_cu();   // blocks of two wavefronts
  uint32_t blocks = (uint32_t)prop.multiProcessorCount * per_cu;
  if (blocks > sim->envs_per_group) blocks = sim->envs_per_group;
  sim->geo_blocks = std::max(1u, blocks);
  sim->snap_blocks = std::max(1u, std::min((uint32_t)prop.multiProcessorCount * 16u, sim->envs_per_group));
  if ((rc = sim->alloc(&sim->d_slots, (size_t)sim->geo_blocks * 2))) return rc;   // one per wavefront

  // ---- per-group queues
  sim->groups.resize(sim->num_groups);
  const size_t n = sim->envs_per_group;
  for (auto& g : sim->groups) {
    for (StepQueues& Q : g.Q) {
      if ((rc = sim->alloc(&Q.counts, kQCounters)) || (rc = sim->alloc(&Q.queries, (size_t)kGeoClasses * 2 * n)) ||
          (rc = sim->alloc(&Q.reset_list, n)))
        return rc;
      Q.stride = (uint32_t)(2 * n);
    }
    if ((rc = sim->alloc(&g.d_actions, n))) return rc;
    HIP_TRY(hipEventCreateWithFlags(&g.moved, hipEventDisableTiming));
    HIP_TRY(hipEventCreateWithFlags(&g.snapped, hipEventDisableTiming));
    HIP_TRY(hipHostMalloc((void**)&g.h_actions, n * sizeof(int64_t), hipHostMallocDefault));
    for (auto& e : g.ev) HIP_TRY(hipEventCreate(&e));
  }
  // the allocation-free entry point's scratch: its address on this device, looked up here so
  // that the entry point itself makes no set-up call
  if ((rc = static_scratch_setup(sim->cfg.gpu_id))) return rc;
  sim->finalized = true;
  if (sim->rotating) {
    // every slot starts loading its next scene right away (simulator.cpp:1573)
    sim->loader = std::thread(loader_loop, sim);
    for (uint32_t i = 0; i < S; ++i) start_scene_swap(sim, i);
  }
  return BPSX_OK;
}

void bpsx_destroy(bpsx_sim* sim) {
  if (!sim) return;
  if (sim->finalized) {
    (void)hipSetDevice(sim->cfg.gpu_id);
    (void)hipDeviceSynchronize();
  }
  if (sim->loader.joinable()) {
    {
      std::lock_guard<std::mutex> lk(sim->loader_mu);
      sim->loader_exit = true;
    }
    sim->loader_cv.notify_all();
    sim->loader.join();
  }
  if (sim->upload_stream) (void)hipStreamDestroy(sim->upload_stream);
  if (sim->side) (void)hipStreamDestroy(sim->side);
  if (sim->h_swap_remaining) (void)hipHostFree(sim->h_swap_remaining);
  for (StepRecord& rec : sim->ring) {
    if (rec.done) (void)hipEventDestroy(rec.done);
    if (rec.remaining) (void)hipHostFree(rec.remaining);
  }
  for (auto& g : sim->groups) {
    if (g.h_actions) (void)hipHostFree(g.h_actions);
    if (g.moved) (void)hipEventDestroy(g.moved);
    if (g.snapped) (void)hipEventDestroy(g.snapped);
    for (auto& e : g.ev)
      if (e) (void)hipEventDestroy(e);
  }
  for (void* p : sim->owned) (void)hipFree(p);
  if (sim->d_batch) (void)hipFree(sim->d_batch);
  delete sim;
}

int bpsx_num_groups(const bpsx_sim* sim, uint32_t* out) {
  if (!sim || !out) return fail(BPSX_E_INVAL, "num_groups: null argument");
  *out = sim->num_groups;
  return BPSX_OK;
}

static int check_group(bpsx_sim* sim, uint32_t group, const char* what) {
  if (!sim) return fail(BPSX_E_INVAL, std::string(what) + ": null simulator");
  if (!sim->finalized) return fail(BPSX_E_STATE, std::string(what) + ": simulator not finalized");
  if (group >= sim->num_groups) return fail(BPSX_E_INVAL, std::string(what) + ": group out of range");
  return BPSX_OK;
}

int bpsx_reset(bpsx_sim* sim, uint32_t group, void* hip_stream) {
  int rc = check_group(sim, group, "reset");
  if (rc) return rc;
  Group& g = sim->groups[group];
  if (g.in_flight) return fail(BPSX_E_STATE, "reset: a step of this group is still in flight");
  HIP_TRY(hipSetDevice(sim->cfg.gpu_id));
  if ((rc = quiesce(sim))) return rc;
  hipStream_t st = (hipStream_t)hip_stream;
  launch_reset(sim->nav, sim->A, g.Q[g.turn], g.Q[g.turn ^ 1], sim->params(group), sim->d_slots, sim->geo_blocks, sim->snap_blocks, st);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipStreamSynchronize(st));
  return BPSX_OK;
}

int bpsx_step_start(bpsx_sim* sim, uint32_t group, const int64_t* actions, int actions_on_device, void* hip_stream) {
  int rc = check_group(sim, group, "step_start");
  if (rc) return rc;
  if (!actions) return fail(BPSX_E_INVAL, "step_start: null actions");
  Group& g = sim->groups[group];
  // the reference aborts with "Not done with previous simulation" (simulator.cpp:1659-1662)
  for (auto& og : sim->groups)
    if (og.in_flight) return fail(BPSX_E_STATE, "step_start: previous step not finished (call step_end first)");
  HIP_TRY(hipSetDevice(sim->cfg.gpu_id));
  hipStream_t st = (hipStream_t)hip_stream;
  // steps that have completed leave the ring; a full ring makes the host wait for its oldest step
  if ((rc = retire_steps(sim, sim->ring_count == kStepRing ? 1 : 0))) return rc;
  const int64_t* d_act = actions;
  if (!actions_on_device) {
    // the staging buffer may still be waiting to be read by a step that has not run yet
    if ((rc = quiesce(sim))) return rc;
    memcpy(g.h_actions, actions, (size_t)sim->envs_per_group * sizeof(int64_t));
    HIP_TRY(hipMemcpyAsync(g.d_actions, g.h_actions, (size_t)sim->envs_per_group * sizeof(int64_t), hipMemcpyHostToDevice, st));
    d_act = g.d_actions;
  }
  if ((rc = rotation_pre_step(sim, st))) return rc;
  g.profiled = sim->profiling;
  StepParams P = sim->params(group);
  P.defer_first_distance = 1;
  launch_step(sim->nav, sim->A, g.Q[g.turn], g.Q[g.turn ^ 1], P, d_act, sim->d_slots, sim->geo_blocks, sim->snap_blocks, st,
              sim->side, g.moved, g.snapped, g.profiled ? g.ev : nullptr);
  g.turn ^= 1;
  HIP_TRY(hipGetLastError());
  g.record = (sim->ring_head + sim->ring_count) % kStepRing;
  StepRecord& rec = sim->ring[g.record];
  rec.ordinal = sim->steps_started;
  // how many envs of each slot are still on a scene that is leaving: read back with the step
  rec.has_remaining = false;
  for (uint32_t slot = 0; slot < sim->cfg.num_active_scenes && !rec.has_remaining; ++slot)
    rec.has_remaining = sim->slots[slot].target != kNoSwap && sim->slots[slot].target != sim->slots[slot].current;
  if (rec.has_remaining)
    HIP_TRY(hipMemcpyAsync(rec.remaining, sim->d_swap_remaining, (size_t)sim->cfg.num_active_scenes * 4, hipMemcpyDeviceToHost, st));
  HIP_TRY(hipEventRecord(rec.done, st));
  sim->ring_count++;
  g.in_flight = true;
  sim->steps_started++;
  sim->env_steps_taken += sim->envs_per_group;
  return BPSX_OK;
}

int bpsx_step_end(bpsx_sim* sim, uint32_t group) {
  int rc = check_group(sim, group, "step_end");
  if (rc) return rc;
  Group& g = sim->groups[group];
  // the reference aborts with "Simulation already done" / group mismatch (simulator.cpp:1679-1689)
  if (!g.in_flight) return fail(BPSX_E_STATE, "step_end: no step in flight for this group");
  // Host-synchronous stepping waits for the step here.  Stream-ordered stepping does not: the
  // step's outputs are complete for whatever is enqueued next on the stream step_start was
  // given, and the host only looks at what earlier steps have brought back.
  if ((rc = retire_steps(sim, (sim->stream_ordered && !g.profiled) ? 0 : sim->ring_count))) return rc;
  g.in_flight = false;
  if (g.profiled) {
    for (int k = 0; k < BPSX_NUM_KERNELS; ++k) {
      float ms = 0;
      HIP_TRY(hipEventElapsedTime(&ms, g.ev[k], g.ev[k + 1]));
      sim->kernel_ms[k] += ms;
    }
    sim->profiled_steps++;
  }
  if (sim->rotating && !sim->loader_error_reported) {
    // a scene that could not be loaded (the reference aborts, simulator.cpp:1723-1726): the step
    // itself is complete, its slot keeps its scene and stops rotating
    std::lock_guard<std::mutex> lk(sim->loader_mu);
    if (!sim->loader_error.empty()) {
      sim->loader_error_reported = true;
      return fail(BPSX_E_UNSUPPORTED, "step_end: scene rotation: loading failed: " + sim->loader_error);
    }
  }
  return BPSX_OK;
}

int bpsx_set_stream_ordered(bpsx_sim* sim, int enabled) {
  if (!sim) return fail(BPSX_E_INVAL, "set_stream_ordered: null simulator");
  for (auto& g : sim->groups)
    if (g.in_flight) return fail(BPSX_E_STATE, "set_stream_ordered: a step is in flight");
  sim->stream_ordered = enabled != 0;
  return BPSX_OK;
}

int bpsx_synchronize(bpsx_sim* sim) {
  if (!sim || !sim->finalized) return fail(BPSX_E_STATE, "synchronize: simulator not finalized");
  HIP_TRY(hipSetDevice(sim->cfg.gpu_id));
  return quiesce(sim);
}

int bpsx_get_outputs(bpsx_sim* sim, uint32_t group, bpsx_outputs* out) {
  int rc = check_group(sim, group, "get_outputs");
  if (rc) return rc;
  if (!out) return fail(BPSX_E_INVAL, "get_outputs: null argument");
  const size_t b = (size_t)group * sim->envs_per_group;
  out->rewards = sim->A.rewards + b;
  out->masks = sim->A.masks + b;
  out->infos = sim->A.infos + b * sim->info_width();
  out->info_width = sim->info_width();
  out->polars = sim->A.polars + b * 2;
  out->n = sim->envs_per_group;
  return BPSX_OK;
}

int bpsx_get_state(bpsx_sim* sim, uint32_t group, bpsx_state* out) {
  int rc = check_group(sim, group, "get_state");
  if (rc) return rc;
  if (!out) return fail(BPSX_E_INVAL, "get_state: null argument");
  const size_t b = (size_t)group * sim->envs_per_group;
  out->position = sim->A.pos + b * 3;
  out->rotation = sim->A.rot + b * 4;
  out->goal = sim->A.goal + b * 3;
  out->poly_ref = sim->A.nav_ref + b;
  out->goal_ref = sim->A.goal_ref + b;
  out->step = sim->A.step + b;
  out->episode = sim->A.episode + b;
  out->num_resets = sim->A.nresets + b;
  out->n = sim->envs_per_group;
  return BPSX_OK;
}

int bpsx_check_errors(bpsx_sim* sim) {
  if (!sim || !sim->finalized) return fail(BPSX_E_STATE, "check_errors: simulator not finalized");
  { const int qrc = quiesce(sim); if (qrc) return qrc; }
  uint32_t f = 0;
  HIP_TRY(hipMemcpy(&f, sim->d_error, 4, hipMemcpyDeviceToHost));
  if (f) return fail(BPSX_E_ACTION, "an action id outside 0..3 was passed to step");
  return BPSX_OK;
}

int bpsx_get_counters(bpsx_sim* sim, uint64_t* out) {
  if (!sim || !sim->finalized || !out) return fail(BPSX_E_STATE, "get_counters: simulator not finalized");
  { const int qrc = quiesce(sim); if (qrc) return qrc; }
  HIP_TRY(hipMemcpy(out, sim->d_counters, BPSX_NUM_COUNTERS * 8, hipMemcpyDeviceToHost));
  return BPSX_OK;
}

int bpsx_set_profiling(bpsx_sim* sim, int enabled) {
  if (!sim) return fail(BPSX_E_INVAL, "set_profiling: null simulator");
  sim->profiling = enabled != 0;
  if (enabled) {
    memset(sim->kernel_ms, 0, sizeof(sim->kernel_ms));
    sim->profiled_steps = 0;
  }
  return BPSX_OK;
}

int bpsx_get_kernel_times(bpsx_sim* sim, double* out_ms_sum, uint64_t* out_steps) {
  if (!sim || !out_ms_sum || !out_steps) return fail(BPSX_E_INVAL, "get_kernel_times: null argument");
  memcpy(out_ms_sum, sim->kernel_ms, sizeof(sim->kernel_ms));
  *out_steps = sim->profiled_steps;
  return BPSX_OK;
}

const char* bpsx_kernel_name(uint32_t idx) { return idx < BPSX_NUM_KERNELS ? kKernelNames[idx] : ""; }

// ---- batched PathFinder-level queries: host arrays in, host arrays out
static int batch_reserve(bpsx_sim* sim, size_t bytes) {
  if (bytes <= sim->batch_bytes) return BPSX_OK;
  if (sim->d_batch) HIP_TRY(hipFree(sim->d_batch));
  sim->d_batch = nullptr;
  sim->batch_bytes = 0;
  HIP_TRY(hipMalloc(&sim->d_batch, bytes));
  sim->batch_bytes = bytes;
  return BPSX_OK;
}
// Brings the host's view of a slot up to date: a swap whose envs have all moved is complete.
static int settle_slot(bpsx_sim* sim, uint32_t slot, uint32_t* remaining_out) {
  SceneSlot& sl = sim->slots[slot];
  uint32_t remaining = 0;
  if (sl.target != kNoSwap) {
    HIP_TRY(hipMemcpy(&remaining, sim->d_swap_remaining + slot, 4, hipMemcpyDeviceToHost));
    if (remaining == 0) {
      // every env is on the new scene: the old one leaves, the slot has no swap any more
      release_scene(sim, sl.current);
      sl.current = sl.target;
      sl.target = kNoSwap;
      const uint32_t none = kNoSwap;
      HIP_TRY(hipMemcpy(sim->d_swap_target + slot, &none, 4, hipMemcpyHostToDevice));
      sim->swaps_completed++;
    }
  }
  if (remaining_out) *remaining_out = remaining;
  return BPSX_OK;
}

int bpsx_swap_scene(bpsx_sim* sim, uint32_t slot, const void* navmesh_bytes, size_t navmesh_size, const float* episodes,
                    uint32_t num_episodes) {
  if (!sim || !sim->finalized) return fail(BPSX_E_STATE, "swap_scene: simulator not finalized");
  if (slot >= sim->cfg.num_active_scenes) return fail(BPSX_E_INVAL, "swap_scene: slot out of range");
  if (!navmesh_bytes) return fail(BPSX_E_INVAL, "swap_scene: null navmesh");
  if (sim->cfg.reset_mode == BPSX_RESET_EPISODES && (!episodes || !num_episodes))
    return fail(BPSX_E_INVAL, "swap_scene: episode-table reset needs at least one episode");
  for (auto& g : sim->groups)
    if (g.in_flight) return fail(BPSX_E_STATE, "swap_scene: a step is in flight");
  if (sim->rotating) return fail(BPSX_E_STATE, "swap_scene: this simulator rotates its scenes by itself");
  HIP_TRY(hipSetDevice(sim->cfg.gpu_id));
  { const int qrc = quiesce(sim); if (qrc) return qrc; }
  // no step is in flight and every earlier one was waited for in step_end: nothing reads the
  // scene that may leave now, and the upload below runs on a stream of its own
  uint32_t remaining = 0;
  int rc = settle_slot(sim, slot, &remaining);
  if (rc) return rc;
  if (remaining) return fail(BPSX_E_STATE, "swap_scene: the previous swap of this slot is still in progress");
  HostScene hs;
  if ((rc = parse_navmesh((const uint8_t*)navmesh_bytes, navmesh_size, &hs))) return rc;
  if (episodes && num_episodes) hs.episodes.assign(episodes, episodes + (size_t)num_episodes * 10);
  SceneSlot& sl = sim->slots[slot];
  const uint32_t S = sim->cfg.num_active_scenes;
  const uint32_t entry = sl.current < S ? slot + S : slot;   // the slot's other table entry
  if ((rc = upload_scene(sim, hs, entry, sim->upload_stream))) return rc;
  const uint32_t per = sim->cfg.num_environments / S;
  HIP_TRY(hipMemcpy(sim->d_swap_remaining + slot, &per, 4, hipMemcpyHostToDevice));
  HIP_TRY(hipMemcpy(sim->d_swap_target + slot, &entry, 4, hipMemcpyHostToDevice));
  sl.target = entry;
  return BPSX_OK;
}

int bpsx_swap_status(bpsx_sim* sim, uint32_t slot, uint32_t* envs_remaining, uint64_t* swaps_completed) {
  if (!sim || !sim->finalized) return fail(BPSX_E_STATE, "swap_status: simulator not finalized");
  if (slot >= sim->cfg.num_active_scenes) return fail(BPSX_E_INVAL, "swap_status: slot out of range");
  for (auto& g : sim->groups)
    if (g.in_flight) return fail(BPSX_E_STATE, "swap_status: a step is in flight");
  HIP_TRY(hipSetDevice(sim->cfg.gpu_id));
  { const int qrc = quiesce(sim); if (qrc) return qrc; }
  uint32_t remaining = 0;
  if (sim->rotating) {
    // as of the last step (step_end keeps the count and completes swaps by itself)
    const SceneSlot& sl = sim->slots[slot];
    remaining = (sl.target != kNoSwap && sl.target != sl.current) ? sim->h_swap_remaining[slot] : 0;
  } else {
    // every slot is brought up to date, so that completed swaps are counted and their old
    // scenes' space is released whichever slot is asked about
    for (uint32_t k = 0; k < sim->cfg.num_active_scenes; ++k) {
      uint32_t rem = 0;
      const int rc = settle_slot(sim, k, &rem);
      if (rc) return rc;
      if (k == slot) remaining = rem;
    }
  }
  if (envs_remaining) *envs_remaining = remaining;
  if (swaps_completed) *swaps_completed = sim->swaps_completed;
  return BPSX_OK;
}

int bpsx_active_scenes(bpsx_sim* sim, uint32_t* out) {
  if (!sim || !sim->finalized || !out) return fail(BPSX_E_STATE, "active_scenes: simulator not finalized");
  for (uint32_t k = 0; k < sim->cfg.num_active_scenes; ++k) {
    const SceneSlot& sl = sim->slots[k];
    // while the slot's next scene is still loading, its envs are on the scene that was drawn before:
    // that scene's index went back to the scenes that are not resident only in name
    out[k] = sl.active_scene;
  }
  return BPSX_OK;
}

int bpsx_rotation_log(bpsx_sim* sim, uint32_t* out, uint32_t max_rows, uint32_t* num_rows) {
  if (!sim || !sim->finalized || !num_rows) return fail(BPSX_E_STATE, "rotation_log: simulator not finalized");
  const uint32_t have = (uint32_t)(sim->rotation_log.size() / 3);
  const uint32_t n = have < max_rows ? have : max_rows;
  if (n && !out) return fail(BPSX_E_INVAL, "rotation_log: null buffer");
  if (n) memcpy(out, sim->rotation_log.data(), (size_t)n * 12);
  sim->rotation_log.erase(sim->rotation_log.begin(), sim->rotation_log.begin() + (long)n * 3);
  *num_rows = n;
  std::lock_guard<std::mutex> lk(sim->loader_mu);
  if (!sim->loader_error.empty()) return fail(BPSX_E_INVAL, "scene rotation: loading failed: " + sim->loader_error);
  return BPSX_OK;
}

int bpsx_swap_stats(bpsx_sim* sim, double* out) {
  if (!sim || !sim->finalized || !out) return fail(BPSX_E_STATE, "swap_stats: simulator not finalized");
  const uint32_t S = sim->cfg.num_active_scenes, per = sim->cfg.num_environments / S;
  out[0] = sim->env_steps_taken ? 100.0 * (double)sim->swaps_completed / (double)sim->env_steps_taken : 0.0;
  // scenes in use and mean envs per scene, summed over the groups like simulator.cpp:1412-1424
  double scenes = 0, mean = 0;
  const uint32_t per_group = S / sim->num_groups;
  for (uint32_t g = 0; g < sim->num_groups; ++g) {
    uint32_t in_use = 0;
    for (uint32_t k = g * per_group; k < (g + 1) * per_group; ++k) {
      const SceneSlot& sl = sim->slots[k];
      const bool moving = sl.target != kNoSwap && sl.target != sl.current;
      const uint32_t rem = moving ? sim->h_swap_remaining[k] : 0;
      in_use += (moving && rem > 0 && rem < per) ? 2u : 1u;
    }
    scenes += in_use;
    mean += (double)sim->envs_per_group / (double)in_use;
  }
  out[1] = scenes;
  out[2] = mean;
  return BPSX_OK;
}

// Batched queries name a scene slot: they see the newest scene uploaded for it.
static uint32_t scene_entry(const bpsx_sim* sim, uint32_t slot) {
  const SceneSlot& sl = sim->slots[slot];
  return sl.target != kNoSwap ? sl.target : sl.current;
}

// wait: the call reads results back on the host, so steps still running on the device are waited
// for first (stream-ordered stepping leaves them running after step_end)
static int check_scene(bpsx_sim* sim, uint32_t scene, const char* what, bool wait = true) {
  if (!sim || !sim->finalized) return fail(BPSX_E_STATE, std::string(what) + ": simulator not finalized");
  if (scene >= sim->cfg.num_active_scenes) return fail(BPSX_E_INVAL, std::string(what) + ": scene out of range");
  for (auto& g : sim->groups)
    if (g.in_flight) return fail(BPSX_E_STATE, std::string(what) + ": a step is in flight");
  HIP_TRY(hipSetDevice(sim->cfg.gpu_id));
  return wait ? quiesce(sim) : BPSX_OK;
}

int bpsx_snap_points(bpsx_sim* sim, uint32_t scene, const float* pts, uint32_t n, float* out_xyz, uint32_t* out_ref) {
  int rc = check_scene(sim, scene, "snap_points");
  if (rc) return rc;
  if (!n) return BPSX_OK;
  if (!pts || !out_xyz || !out_ref) return fail(BPSX_E_INVAL, "snap_points: null argument");
  const size_t f3 = (size_t)n * 12;
  if ((rc = batch_reserve(sim, 2 * f3 + (size_t)n * 4))) return rc;
  char* b = (char*)sim->d_batch;
  float* d_in = (float*)b; float* d_xyz = (float*)(b + f3); uint32_t* d_ref = (uint32_t*)(b + 2 * f3);
  HIP_TRY(hipMemcpy(d_in, pts, f3, hipMemcpyHostToDevice));
  launch_snap_batch(sim->nav, scene_entry(sim, scene), d_in, n, d_xyz, d_ref, sim->snap_blocks * 4, nullptr);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipMemcpy(out_xyz, d_xyz, f3, hipMemcpyDeviceToHost));
  HIP_TRY(hipMemcpy(out_ref, d_ref, (size_t)n * 4, hipMemcpyDeviceToHost));
  return BPSX_OK;
}

int bpsx_try_steps(bpsx_sim* sim, uint32_t scene, const float* start_xyz, const uint32_t* start_ref, const float* end_xyz,
                   uint32_t n, float* out_xyz, uint32_t* out_ref) {
  int rc = check_scene(sim, scene, "try_steps");
  if (rc) return rc;
  if (!n) return BPSX_OK;
  if (!start_xyz || !start_ref || !end_xyz || !out_xyz || !out_ref) return fail(BPSX_E_INVAL, "try_steps: null argument");
  const size_t f3 = (size_t)n * 12, u1 = (size_t)n * 4;
  if ((rc = batch_reserve(sim, 3 * f3 + 2 * u1))) return rc;
  char* b = (char*)sim->d_batch;
  float* d_s = (float*)b; float* d_e = (float*)(b + f3); float* d_o = (float*)(b + 2 * f3);
  uint32_t* d_sr = (uint32_t*)(b + 3 * f3); uint32_t* d_or = (uint32_t*)(b + 3 * f3 + u1);
  HIP_TRY(hipMemcpy(d_s, start_xyz, f3, hipMemcpyHostToDevice));
  HIP_TRY(hipMemcpy(d_e, end_xyz, f3, hipMemcpyHostToDevice));
  HIP_TRY(hipMemcpy(d_sr, start_ref, u1, hipMemcpyHostToDevice));
  launch_try_step_batch(sim->nav, scene_entry(sim, scene), d_s, d_sr, d_e, n, d_o, d_or, nullptr);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipMemcpy(out_xyz, d_o, f3, hipMemcpyDeviceToHost));
  HIP_TRY(hipMemcpy(out_ref, d_or, u1, hipMemcpyDeviceToHost));
  return BPSX_OK;
}

int bpsx_geodesic(bpsx_sim* sim, uint32_t scene, const float* start_xyz, const uint32_t* start_ref, const float* end_xyz,
                  const uint32_t* end_ref, uint32_t n, float* out_dist) {
  int rc = check_scene(sim, scene, "geodesic");
  if (rc) return rc;
  if (!n) return BPSX_OK;
  if (!start_xyz || !start_ref || !end_xyz || !end_ref || !out_dist) return fail(BPSX_E_INVAL, "geodesic: null argument");
  const size_t f3 = (size_t)n * 12, u1 = (size_t)n * 4, qb = (size_t)n * sizeof(GeoQuery);
  if ((rc = batch_reserve(sim, 2 * f3 + 3 * u1 + qb + 64))) return rc;
  char* b = (char*)sim->d_batch;
  GeoQuery* d_q = (GeoQuery*)b;  // first: keeps the 4-byte members aligned trivially
  float* d_s = (float*)(b + qb); float* d_e = (float*)(b + qb + f3);
  uint32_t* d_sr = (uint32_t*)(b + qb + 2 * f3); uint32_t* d_er = (uint32_t*)(b + qb + 2 * f3 + u1);
  float* d_o = (float*)(b + qb + 2 * f3 + 2 * u1);
  HIP_TRY(hipMemcpy(d_s, start_xyz, f3, hipMemcpyHostToDevice));
  HIP_TRY(hipMemcpy(d_e, end_xyz, f3, hipMemcpyHostToDevice));
  HIP_TRY(hipMemcpy(d_sr, start_ref, u1, hipMemcpyHostToDevice));
  HIP_TRY(hipMemcpy(d_er, end_ref, u1, hipMemcpyHostToDevice));
  launch_geodesic_batch(sim->nav, scene_entry(sim, scene), d_s, d_sr, d_e, d_er, n, d_q, sim->d_batch_counts, d_o, sim->d_slots,
                        sim->geo_blocks, sim->d_counters, nullptr);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipMemcpy(out_dist, d_o, u1, hipMemcpyDeviceToHost));
  return BPSX_OK;
}

int bpsx_geodesic_static(bpsx_sim* sim, uint32_t scene, const float* start_xyz, const uint32_t* start_ref,
                         const float* end_xyz, const uint32_t* end_ref, uint32_t n, float* out_dist, void* hip_stream) {
  int rc = check_scene(sim, scene, "geodesic_static", false);   // stream-ordered: nothing is waited for
  if (rc) return rc;
  if (n > BPSX_STATIC_MAX_QUERIES)
    return fail(BPSX_E_INVAL, "geodesic_static: n = " + std::to_string(n) + " exceeds BPSX_STATIC_MAX_QUERIES = " +
                                  std::to_string(BPSX_STATIC_MAX_QUERIES));
  if (!n) return BPSX_OK;
  if (!start_xyz || !start_ref || !end_xyz || !end_ref || !out_dist) return fail(BPSX_E_INVAL, "geodesic_static: null argument");
  unsigned char* base = g_static_scratch[sim->cfg.gpu_id];   // set up by bpsx_finalize on this device
  if (!base) return fail(BPSX_E_STATE, "geodesic_static: the static scratch array was not set up on this device");
  GeoQuery* d_q = (GeoQuery*)base;
  uint32_t* d_counts = (uint32_t*)(base + kStaticQueriesBytes);
  GeoSlot* d_slots = (GeoSlot*)(base + kStaticQueriesBytes + kStaticCountsBytes);
  // The counters are rewritten by a kernel at the start of every call; node pools and queries
  // are written before they are read.  Nothing else of the previous call's contents is used.
  launch_geodesic_batch(sim->nav, scene_entry(sim, scene), start_xyz, start_ref, end_xyz, end_ref, n, d_q, d_counts, out_dist,
                        d_slots, std::min(kStaticBlocks, std::max(1u, (n + 1) / 2)), sim->d_counters, (hipStream_t)hip_stream);
  HIP_TRY(hipGetLastError());
  return BPSX_OK;
}

int bpsx_random_points(bpsx_sim* sim, uint32_t scene, const float* u, uint32_t n, float* out_xyz, uint32_t* out_ref) {
  int rc = check_scene(sim, scene, "random_points");
  if (rc) return rc;
  if (!n) return BPSX_OK;
  if (!u || !out_xyz || !out_ref) return fail(BPSX_E_INVAL, "random_points: null argument");
  const size_t f3 = (size_t)n * 12;
  if ((rc = batch_reserve(sim, 2 * f3 + (size_t)n * 4))) return rc;
  char* b = (char*)sim->d_batch;
  float* d_in = (float*)b; float* d_xyz = (float*)(b + f3); uint32_t* d_ref = (uint32_t*)(b + 2 * f3);
  HIP_TRY(hipMemcpy(d_in, u, f3, hipMemcpyHostToDevice));
  launch_random_points(sim->nav, scene_entry(sim, scene), d_in, n, d_xyz, d_ref, nullptr);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipMemcpy(out_xyz, d_xyz, f3, hipMemcpyDeviceToHost));
  HIP_TRY(hipMemcpy(out_ref, d_ref, (size_t)n * 4, hipMemcpyDeviceToHost));
  return BPSX_OK;
}

}  // extern "C"
