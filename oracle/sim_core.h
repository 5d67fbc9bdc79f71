// TEST INFRASTRUCTURE — CPU restatement of the reference's per-agent state machine and of
// its worker-thread dispatch, templated on the navmesh backend so that the same code drives
// both the independent restatement (nav_oracle) and the compiled reference PathFinder
// (oracle/_ref).  simulator.cpp cannot be compiled (bps3D, glm, simdjson, pybind11 are
// absent), so this file follows it by reading:
//   BaseSimulator::reset/step/handleMovement/updateObservationState  simulator.cpp:601-710
//   PointNav::InfoFunctor / RewardFunctor                            simulator.cpp:737-825
//   Flee::InfoFunctor / RewardFunctor                                simulator.cpp:830-887
//   Exploration::InfoFunctor / RewardFunctor                         simulator.cpp:889-997
//   computeGeoDist                                                   simulator.cpp:553-563
//   RolloutGenerator::simulate / simulateStart / simulateEnd         simulator.cpp:1619-1700
//   EnvironmentGroup env->scene assignment                           simulator.cpp:1205-1221
//   scene rotation (SceneSwapper, SceneTracker, swapReady/swapScene)  simulator.cpp:1063-1178, 1284-1310, 1636-1642
//     (the reference loads the next scene in a background thread and picks it at random; here
//      the caller names it, like the engine's bpsx_swap_scene)
// glm closed forms (angleAxis, quat*quat, quat*vec3, mat3_cast) are written out; glm is
// not vendored by the reference, so those are "parity unpinned" and pinned here by closed
// forms in tests/test_oracle_closed_forms.py.  The same holds for glm::inverse(quat) =
// conjugate / dot with dot = (w*w + x*x) + (y*y + z*z) (glm 0.9.9 compute_dot for quaternions),
// used by the Exploration task: parity unpinned, pinned by closed forms.
//
// Deviation by design: the reference draws the reset episode from a per-thread mt19937
// claimed racily by worker threads (simulator.cpp:605-607, 1626, 1736); this build defines a
// counter-based stream keyed by (seed, env index, reset count) so resets are reproducible.
#pragma once
#include <array>
#include <atomic>
#include <cmath>
#include <condition_variable>
#include <cstdint>
#include <cstring>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

namespace simcore {

constexpr float SUCCESS_REWARD = 2.5f;
constexpr float SLACK_REWARD = 1e-2f;
constexpr float SUCCESS_DISTANCE = 0.2f;
constexpr float FORWARD_STEP_SIZE = 0.25f;
enum Task : uint32_t { TASK_POINTNAV = 0, TASK_FLEE = 1, TASK_EXPLORATION = 2 };

struct NavPt {
  float xyz[3];
  uint32_t ref;
};

// ---- counter-based stream shared by every implementation of the engine
inline uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
inline uint64_t reset_key(uint64_t seed, uint32_t env, uint32_t reset_count) {
  return mix64(seed + 0x9E3779B97F4A7C15ull * ((uint64_t)env + 1) + 0xD1B54A32D192ED03ull * ((uint64_t)reset_count + 1));
}
// k-th 32-bit draw of a reset
inline uint32_t reset_draw(uint64_t key, uint32_t k) { return (uint32_t)(mix64(key + 0x9E3779B97F4A7C15ull * ((uint64_t)k + 1)) >> 32); }
inline uint32_t draw_index(uint32_t r, uint32_t n) { return (uint32_t)(((uint64_t)r * (uint64_t)n) >> 32); }
inline float draw_unit(uint32_t r) { return (float)(r >> 8) * (1.0f / 16777216.0f); }  // [0,1), 24 bits

// ---- glm closed forms (quaternions stored x,y,z,w)
inline void quat_mul(const float* p, const float* q, float* o) {
  const float w = p[3] * q[3] - p[0] * q[0] - p[1] * q[1] - p[2] * q[2];
  const float x = p[3] * q[0] + p[0] * q[3] + p[1] * q[2] - p[2] * q[1];
  const float y = p[3] * q[1] + p[1] * q[3] + p[2] * q[0] - p[0] * q[2];
  const float z = p[3] * q[2] + p[2] * q[3] + p[0] * q[1] - p[1] * q[0];
  o[0] = x; o[1] = y; o[2] = z; o[3] = w;
}
inline void cross3(const float* a, const float* b, float* o) {
  o[0] = a[1] * b[2] - b[1] * a[2];
  o[1] = a[2] * b[0] - b[2] * a[0];
  o[2] = a[0] * b[1] - b[0] * a[1];
}
inline void quat_rotate(const float* q, const float* v, float* o) {
  float uv[3], uuv[3];
  cross3(q, v, uv);
  cross3(q, uv, uuv);
  for (int k = 0; k < 3; ++k) o[k] = v[k] + ((uv[k] * q[3]) + uuv[k]) * 2.0f;
}
// v_view = transpose(mat3_cast(q)) * v
inline void view_from_world(const float* q, const float* v, float* o) {
  const float qxx = q[0] * q[0], qyy = q[1] * q[1], qzz = q[2] * q[2];
  const float qxz = q[0] * q[2], qxy = q[0] * q[1], qyz = q[1] * q[2];
  const float qwx = q[3] * q[0], qwy = q[3] * q[1], qwz = q[3] * q[2];
  const float m00 = 1.0f - 2.0f * (qyy + qzz), m01 = 2.0f * (qxy + qwz), m02 = 2.0f * (qxz - qwy);
  const float m10 = 2.0f * (qxy - qwz), m11 = 1.0f - 2.0f * (qxx + qzz), m12 = 2.0f * (qyz + qwx);
  const float m20 = 2.0f * (qxz + qwy), m21 = 2.0f * (qyz - qwx), m22 = 1.0f - 2.0f * (qxx + qyy);
  // column c of mat3_cast is (mc0, mc1, mc2); the transposed product dots v with columns
  o[0] = m00 * v[0] + m01 * v[1] + m02 * v[2];
  o[1] = m10 * v[0] + m11 * v[1] + m12 * v[2];
  o[2] = m20 * v[0] + m21 * v[1] + m22 * v[2];
}
struct TurnConstants {
  float left[4], right[4];
  TurnConstants() {
    const float a = 10.0f * 0.01745329251994329576923690768489f;  // glm::radians(10.f)
    const float s = sinf(a * 0.5f), c = cosf(a * 0.5f);
    left[0] = 0; left[1] = s; left[2] = 0; left[3] = c;
    const float sn = sinf(-a * 0.5f), cn = cosf(-a * 0.5f);
    right[0] = 0; right[1] = sn; right[2] = 0; right[3] = cn;
  }
};

struct Env {
  uint32_t scene = 0;   // index into the simulator's scene list
  uint32_t slot = 0;    // scene slot the env belongs to (fixed)
  float pos[3] = {0, 0, 0}, rot[4] = {0, 0, 0, 1}, goal[3] = {0, 0, 0};
  NavPt nav{{0, 0, 0}, 0}, navGoal{{0, 0, 0}, 0};
  uint32_t step = 0;
  bool updated = false;
  float infoPrevDist = 0, cumDist = 0, initDist = 0, prevPos[3] = {0, 0, 0};
  float rewardPrevDist = 0;
  uint32_t episode = 0, numResets = 0;
  // Exploration: cells visited, in the frame of the episode's start pose
  float initPos[3] = {0, 0, 0}, invInitRot[4] = {0, 0, 0, 1};
  std::vector<std::array<int, 3>> visited;
};
// glm::inverse(quat): conjugate(q) / dot(q, q)
inline void quat_inverse(const float* q, float* o) {
  const float d = (q[3] * q[3] + q[0] * q[0]) + (q[1] * q[1] + q[2] * q[2]);
  o[3] = q[3] / d; o[0] = -q[0] / d; o[1] = -q[1] / d; o[2] = -q[2] / d;
}

struct SceneEpisodes {
  std::vector<float> rows;  // [E][10]
  uint32_t count = 0;
};

// Backend concept:
//   struct B { struct Scene; struct Ctx;
//     static std::shared_ptr<Scene> load(const uint8_t*, size_t, std::string* err);
//     static std::unique_ptr<Ctx> make_ctx(const std::vector<std::shared_ptr<Scene>>&);  // one per thread
//     NavPt Ctx::snap(uint32_t scene, const float* p);
//     NavPt Ctx::tryStep(uint32_t scene, const NavPt& s, const float* end);
//     float Ctx::geodesic(uint32_t scene, const NavPt& a, const NavPt& b);
//     bool  Ctx::sample(uint32_t scene, float u0, float s, float t, float* xyz); }
template <class B>
class Sim {
 public:
  Sim(uint32_t numEnvs, uint32_t numScenes, bool doubleBuffered, uint32_t resetMode, uint64_t seed,
      uint32_t maxSteps, int numThreads)
      : numEnvs_(numEnvs), numScenes_(numScenes), groups_(doubleBuffered ? 2 : 1), resetMode_(resetMode),
        seed_(seed), maxSteps_(maxSteps ? maxSteps : 500), numThreads_(numThreads < 1 ? 1 : numThreads) {}
  ~Sim() { stopWorkers(); }
  void setTask(uint32_t task) { task_ = task; }
  // Starts a swap of scene slot `slot`: its envs move to the new scene when their episode ends.
  // False while the previous swap of the slot is in progress.
  bool swapScene(uint32_t slot, const uint8_t* bytes, size_t n, const float* episodes, uint32_t numEpisodes,
                 std::string* err) {
    if (slot >= numScenes_) { *err = "slot out of range"; return false; }
    if (swapRemaining_[slot]) { *err = "previous swap still in progress"; return false; }
    auto sc = B::load(bytes, n, err);
    if (!sc) return false;
    scenes_.push_back(sc);
    SceneEpisodes e;
    e.count = numEpisodes;
    e.rows.assign(episodes, episodes + (size_t)numEpisodes * 10);
    episodes_.push_back(std::move(e));
    swapTarget_[slot] = (uint32_t)scenes_.size() - 1;
    swapRemaining_[slot] = numEnvs_ / numScenes_;
    // the query contexts are per thread and per scene: rebuild them with the new scene
    std::vector<std::thread> builders;
    for (int t = 0; t < numThreads_; ++t) builders.emplace_back([this, t] { ctxs_[t] = B::make_ctx(scenes_); });
    for (auto& b : builders) b.join();
    return true;
  }
  uint32_t swapRemaining(uint32_t slot) const { return slot < numScenes_ ? swapRemaining_[slot].load() : 0; }

  bool addScene(const uint8_t* bytes, size_t n, const float* episodes, uint32_t numEpisodes, std::string* err) {
    auto s = B::load(bytes, n, err);
    if (!s) return false;
    scenes_.push_back(s);
    SceneEpisodes e;
    e.count = numEpisodes;
    e.rows.assign(episodes, episodes + (size_t)numEpisodes * 10);
    episodes_.push_back(std::move(e));
    return true;
  }
  bool finalize(std::string* err) {
    if (scenes_.size() != numScenes_) { *err = "scene count differs from num_active_scenes"; return false; }
    if (!numEnvs_ || numEnvs_ % numScenes_ != 0 || numScenes_ % groups_ != 0) {
      *err = "num_environments must be a multiple of num_active_scenes, and scenes of groups";
      return false;
    }
    envsPerGroup_ = numEnvs_ / groups_;
    // group g owns scenes [g*S/G, (g+1)*S/G) and, per scene, a contiguous block of N/S envs
    envs_.assign(numEnvs_, Env());
    const uint32_t envsPerScene = numEnvs_ / numScenes_;
    for (uint32_t i = 0; i < numEnvs_; ++i) { envs_[i].scene = i / envsPerScene; envs_[i].slot = i / envsPerScene; }
    swapTarget_.assign(numScenes_, 0xffffffffu);
    swapRemaining_ = std::vector<std::atomic<uint32_t>>(numScenes_);
    for (auto& r : swapRemaining_) r.store(0);
    rewards_.assign(numEnvs_, 0.f);
    masks_.assign(numEnvs_, 0);
    infos_.assign((size_t)numEnvs_ * 3, 0.f);
    polars_.assign((size_t)numEnvs_ * 2, 0.f);
    // every participant builds its own query contexts, concurrently, like the reference's
    // worker threads do at start-up (simulator.cpp:1712-1738)
    ctxs_.resize((size_t)numThreads_);
    {
      std::vector<std::thread> builders;
      for (int t = 0; t < numThreads_; ++t) builders.emplace_back([this, t] { ctxs_[t] = B::make_ctx(scenes_); });
      for (auto& b : builders) b.join();
    }
    startWorkers();
    return true;
  }
  uint32_t envsPerGroup() const { return envsPerGroup_; }
  uint32_t numGroups() const { return groups_; }

  void reset(uint32_t group) { run(group, nullptr, true); }
  void step(uint32_t group, const int64_t* actions) { run(group, actions, false); }

  Env& env(uint32_t group, uint32_t i) { return envs_[(size_t)group * envsPerGroup_ + i]; }
  float* rewards(uint32_t g) { return &rewards_[(size_t)g * envsPerGroup_]; }
  uint8_t* masks(uint32_t g) { return &masks_[(size_t)g * envsPerGroup_]; }
  float* infos(uint32_t g) { return &infos_[(size_t)g * envsPerGroup_ * 3]; }
  float* polars(uint32_t g) { return &polars_[(size_t)g * envsPerGroup_ * 2]; }
  typename B::Ctx& ctx(int t) { return *ctxs_[t]; }
  int numThreads() const { return numThreads_; }
  bool sawBadAction() const { return badAction_.load(); }

 private:
  // ------------------------------------------------------------ per-agent logic
  void updateObservation(uint32_t gi) {
    Env& e = envs_[gi];
    const float toGoal[3] = {e.goal[0] - e.pos[0], e.goal[1] - e.pos[1], e.goal[2] - e.pos[2]};
    float v[3];
    view_from_world(e.rot, toGoal, v);
    const float x = -v[2], y = v[0];
    polars_[(size_t)gi * 2 + 0] = sqrtf(x * x + y * y);
    polars_[(size_t)gi * 2 + 1] = -atan2f(y, x);
  }
  void resetEnv(uint32_t gi, typename B::Ctx& c) {
    Env& e = envs_[gi];
    e.step = 1;
    const uint64_t key = reset_key(seed_, gi, e.numResets);
    e.numResets++;
    float ep[10];
    if (resetMode_ == 0) {
      const SceneEpisodes& se = episodes_[e.scene];
      e.episode = draw_index(reset_draw(key, 0), se.count);
      memcpy(ep, &se.rows[(size_t)e.episode * 10], sizeof(ep));
    } else {
      // sampled reset: start, goal by area-weighted sampling; heading = k left turns
      e.episode = 0;
      float sxyz[3] = {0, 0, 0}, gxyz[3] = {0, 0, 0};
      c.sample(e.scene, draw_unit(reset_draw(key, 0)), draw_unit(reset_draw(key, 1)), draw_unit(reset_draw(key, 2)), sxyz);
      c.sample(e.scene, draw_unit(reset_draw(key, 3)), draw_unit(reset_draw(key, 4)), draw_unit(reset_draw(key, 5)), gxyz);
      const uint32_t k = draw_index(reset_draw(key, 6), 36);
      float q[4] = {0, 0, 0, 1};
      for (uint32_t i = 0; i < k; ++i) quat_mul(q, turns_.left, q);
      memcpy(ep, sxyz, 12); memcpy(ep + 3, q, 16); memcpy(ep + 7, gxyz, 12);
    }
    memcpy(e.pos, ep, 12);
    memcpy(e.rot, ep + 3, 16);
    memcpy(e.goal, ep + 7, 12);
    e.nav = c.snap(e.scene, e.pos);
    updateObservation(gi);
    if (task_ == TASK_FLEE) {
      // Flee::InfoFunctor::reset: the start point is kept where PointNav keeps the goal point
      e.navGoal = e.nav;
      e.infoPrevDist = 0.0f;
      e.rewardPrevDist = 0.0f;
      return;
    }
    if (task_ == TASK_EXPLORATION) {
      e.navGoal = NavPt{{0, 0, 0}, 0};
      e.visited.clear();
      memcpy(e.initPos, e.pos, 12);
      quat_inverse(e.rot, e.invInitRot);
      visit(e);
      e.infoPrevDist = (float)(e.visited.size() - 1);
      e.rewardPrevDist = e.infoPrevDist;
      return;
    }
    // InfoFunctor::reset
    e.navGoal = c.snap(e.scene, e.goal);
    e.cumDist = 0;
    e.initDist = c.geodesic(e.scene, e.nav, e.navGoal);
    e.infoPrevDist = e.initDist;
    memcpy(e.prevPos, e.pos, 12);
    // RewardFunctor::reset
    e.rewardPrevDist = e.infoPrevDist;
  }
  // Exploration::InfoFunctor::update
  static void visit(Env& e) {
    const float d[3] = {e.pos[0] - e.initPos[0], e.pos[1] - e.initPos[1], e.pos[2] - e.initPos[2]};
    float g[3];
    quat_rotate(e.invInitRot, d, g);
    // int(x) as x86 converts it: INT32_MIN for NaN and for values no int32 holds
    auto toCell = [](float x) { return (x > -2147483648.0f && x < 2147483648.0f) ? (int)x : (int)0x80000000; };
    const std::array<int, 3> cell = {toCell(g[0] / 1.0f), toCell(g[1] / 1.0f), toCell(g[2] / 1.0f)};
    for (const auto& v : e.visited)
      if (v == cell) return;
    e.visited.push_back(cell);
  }
  bool stepEnv(uint32_t gi, int64_t action, typename B::Ctx& c) {
    Env& e = envs_[gi];
    if (action < 0 || action > 3) {
      // the reference aborts (simulator.cpp:704-708); the engine flags it and leaves the agent alone
      badAction_.store(true);
      return false;
    }
    e.step++;
    bool done = (float)e.step >= (float)maxSteps_;
    e.updated = false;
    if (action == 0) {
      done = true;
    } else {
      if (action == 1) {
        const float fwd[3] = {0.f * FORWARD_STEP_SIZE, 0.f * FORWARD_STEP_SIZE, -1.f * FORWARD_STEP_SIZE};
        float delta[3];
        quat_rotate(e.rot, fwd, delta);
        const float np[3] = {e.pos[0] + delta[0], e.pos[1] + delta[1], e.pos[2] + delta[2]};
        e.nav = c.tryStep(e.scene, e.nav, np);
        memcpy(e.pos, e.nav.xyz, 12);
        e.updated = true;
      } else if (action == 2) {
        quat_mul(e.rot, turns_.left, e.rot);
      } else {
        quat_mul(e.rot, turns_.right, e.rot);
      }
      updateObservation(gi);
    }
    if (task_ != TASK_POINTNAV) {
      float v;
      if (task_ == TASK_FLEE) {
        if (e.updated) e.infoPrevDist = c.geodesic(e.scene, e.navGoal, e.nav);
        v = e.infoPrevDist;
        rewards_[gi] = v - e.rewardPrevDist;
      } else {
        if (e.updated) visit(e);
        v = (float)(e.visited.size() - 1);
        rewards_[gi] = (float)(0.25 * (double)(v - e.rewardPrevDist));
      }
      e.rewardPrevDist = v;
      masks_[gi] = done ? 0 : 1;
      infos_[(size_t)gi * 3 + 0] = v;
      infos_[(size_t)gi * 3 + 1] = 0;
      infos_[(size_t)gi * 3 + 2] = 0;
      return done;
    }
    // InfoFunctor::step
    float dist = 0, success = 0, spl = 0;
    if (done) {
      dist = c.geodesic(e.scene, e.navGoal, e.nav);
      success = (dist < SUCCESS_DISTANCE) ? 1.0f : 0.0f;
      const float mx = e.initDist < e.cumDist ? e.cumDist : e.initDist;  // std::max(a, b) = (a < b) ? b : a
      spl = success * e.initDist / mx;
    } else if (e.updated) {
      dist = c.geodesic(e.scene, e.navGoal, e.nav);
      const float dx = e.pos[0] - e.prevPos[0], dy = e.pos[1] - e.prevPos[1], dz = e.pos[2] - e.prevPos[2];
      e.cumDist += sqrtf(dx * dx + dy * dy + dz * dz);
      e.infoPrevDist = dist;
      memcpy(e.prevPos, e.pos, 12);
    } else {
      dist = e.infoPrevDist;
    }
    // RewardFunctor::step
    float reward = -SLACK_REWARD;
    if (done) reward += SUCCESS_REWARD * spl;
    else reward += e.rewardPrevDist - dist;
    e.rewardPrevDist = dist;
    rewards_[gi] = reward;
    masks_[gi] = done ? 0 : 1;
    infos_[(size_t)gi * 3 + 0] = success;
    infos_[(size_t)gi * 3 + 1] = spl;
    infos_[(size_t)gi * 3 + 2] = dist;
    return done;
  }

  // ------------------------------------------------------------ dispatch
  void simulate(int tid) {
    typename B::Ctx& c = *ctxs_[tid];
    const uint32_t base = curGroup_ * envsPerGroup_;
    for (;;) {
      const uint32_t i = nextEnv_.fetch_add(1, std::memory_order_acq_rel);
      if (i >= envsPerGroup_) break;
      const uint32_t gi = base + i;
      if (curReset_) {
        resetEnv(gi, c);
      } else if (stepEnv(gi, curActions_[i], c)) {
        Env& e = envs_[gi];
        const uint32_t tgt = swapTarget_[e.slot];
        if (tgt != 0xffffffffu && e.scene != tgt) {   // swapReady / swapScene
          e.scene = tgt;
          swapRemaining_[e.slot].fetch_sub(1);
        }
        resetEnv(gi, c);
      }
    }
  }
  void run(uint32_t group, const int64_t* actions, bool isReset) {
    curGroup_ = group; curActions_ = actions; curReset_ = isReset;
    nextEnv_.store(0, std::memory_order_release);
    finished_.store(0, std::memory_order_release);
    {
      std::lock_guard<std::mutex> lk(mu_);
      generation_++;
    }
    cv_.notify_all();
    simulate(0);
    while (finished_.load(std::memory_order_acquire) != numThreads_ - 1) {
#if defined(__x86_64__)
      __builtin_ia32_pause();
#endif
    }
  }
  void startWorkers() {
    for (int t = 1; t < numThreads_; ++t)
      workers_.emplace_back([this, t] {
        uint64_t seen = 0;
        for (;;) {
          {
            std::unique_lock<std::mutex> lk(mu_);
            cv_.wait(lk, [&] { return generation_ != seen || quit_; });
            if (quit_) return;
            seen = generation_;
          }
          simulate(t);
          finished_.fetch_add(1, std::memory_order_acq_rel);
        }
      });
  }
  void stopWorkers() {
    {
      std::lock_guard<std::mutex> lk(mu_);
      quit_ = true;
    }
    cv_.notify_all();
    for (auto& w : workers_) w.join();
    workers_.clear();
  }

  uint32_t task_ = TASK_POINTNAV;
  std::vector<uint32_t> swapTarget_;
  std::vector<std::atomic<uint32_t>> swapRemaining_;
  uint32_t numEnvs_, numScenes_, groups_, resetMode_;
  uint64_t seed_;
  uint32_t maxSteps_;
  int numThreads_;
  uint32_t envsPerGroup_ = 0;
  TurnConstants turns_;
  std::vector<std::shared_ptr<typename B::Scene>> scenes_;
  std::vector<SceneEpisodes> episodes_;
  std::vector<Env> envs_;
  std::vector<float> rewards_, infos_, polars_;
  std::vector<uint8_t> masks_;
  std::vector<std::unique_ptr<typename B::Ctx>> ctxs_;
  std::vector<std::thread> workers_;
  std::mutex mu_;
  std::condition_variable cv_;
  uint64_t generation_ = 0;
  bool quit_ = false;
  std::atomic<uint32_t> nextEnv_{0};
  std::atomic<int> finished_{0};
  std::atomic<bool> badAction_{false};
  uint32_t curGroup_ = 0;
  const int64_t* curActions_ = nullptr;
  bool curReset_ = false;
};

}  // namespace simcore
