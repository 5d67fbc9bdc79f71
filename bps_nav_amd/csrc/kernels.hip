// HIP kernels of the batch environment step (gfx950) and their launch wrappers.
//
// One step of a group of n agents is four launches:
//   step_move      lane per agent: action, turn / forward move with wall sliding, polar
//                  observation, and a geodesic query (goal -> agent) when the agent moved or
//                  the episode ended; an agent whose episode ended also picks its next episode
//                  here and is queued for reset (simulator.cpp:620-632, 651-710, 601-610)
//   reset_snap     two wavefronts per queued agent: snap start and goal of the new episode,
//                  polar, and the new episode's first query (agent -> goal)
//                                                        (simulator.cpp:611-614, 744-751)
//   geodesic       wavefront per query, both kinds in one launch: A* + funnel; blocks of two
//                  wavefronts so that the longest searches can take a block's whole LDS
//                                                        (PathFinder.cpp:485-541)
//   step_finish    lane per agent: info, reward, mask from the terminal transition, then the
//                  new episode's distance bookkeeping    (simulator.cpp:634-641, 758-822, 749-755)
// In a step, reset_snap runs on a second stream next to geodesic: the first query of an episode
// that begins in step t is answered by step t + 1's geodesic launch, and its result enters the
// bookkeeping at the start of step t + 1's step_finish.  No output of step t depends on it (the
// reference computes it inside the reset and uses it from the next step on).  A reset of a
// whole group (bpsx_reset) runs the four launches in order, first queries included.
// The Flee and Exploration tasks (simulator.cpp:830-997) run through the same four launches:
// Flee keeps the episode's start point where PointNav keeps the snapped goal, so its
// "distance from start" is the same start-point -> agent query; Exploration makes no queries
// and keeps its visited cells per agent in HBM.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "../../include/bpsx.h"
#include "geodesic_device.h"
// A second instantiation of the same search for the few longest queries of a step: all 2048
// link words, twice the window and twice the hash heads in LDS.  Such a query takes the LDS of a
// whole two-wavefront block (see k_geodesic).
#undef BPSX_GEO_NS
#undef BPSX_LINKS_LDS
#undef BPSX_HEAP_LDS
#undef BPSX_WINDOW
#undef BPSX_HASH
#define BPSX_GEO_NS geo_long
#define BPSX_LINKS_LDS 2048
#define BPSX_HEAP_LDS 32
#define BPSX_WINDOW 256
#define BPSX_HASH 1024
#include "geodesic_device.h"
#include "kernels.h"

namespace bpsx {

namespace {

// ---- counter-based reset stream (identical integer arithmetic on host and device)
BPSX_DEV uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
BPSX_DEV uint64_t reset_key(uint64_t seed, uint32_t env, uint32_t count) {
  return mix64(seed + 0x9E3779B97F4A7C15ull * ((uint64_t)env + 1) + 0xD1B54A32D192ED03ull * ((uint64_t)count + 1));
}
BPSX_DEV uint32_t reset_draw(uint64_t key, uint32_t k) {
  return (uint32_t)(mix64(key + 0x9E3779B97F4A7C15ull * ((uint64_t)k + 1)) >> 32);
}
BPSX_DEV uint32_t draw_index(uint32_t r, uint32_t n) { return (uint32_t)(((uint64_t)r * (uint64_t)n) >> 32); }
BPSX_DEV float draw_unit(uint32_t r) { return (float)(r >> 8) * (1.0f / 16777216.0f); }

// ---- glm closed forms, quaternions stored x,y,z,w
BPSX_DEV void quat_mul(const float* p, const float* q, float* o) {
  const float w = p[3] * q[3] - p[0] * q[0] - p[1] * q[1] - p[2] * q[2];
  const float x = p[3] * q[0] + p[0] * q[3] + p[1] * q[2] - p[2] * q[1];
  const float y = p[3] * q[1] + p[1] * q[3] + p[2] * q[0] - p[0] * q[2];
  const float z = p[3] * q[2] + p[2] * q[3] + p[0] * q[1] - p[1] * q[0];
  o[0] = x; o[1] = y; o[2] = z; o[3] = w;
}
BPSX_DEV void cross3(const float* a, const float* b, float* o) {
  o[0] = a[1] * b[2] - b[1] * a[2];
  o[1] = a[2] * b[0] - b[2] * a[0];
  o[2] = a[0] * b[1] - b[0] * a[1];
}
BPSX_DEV void quat_rotate(const float* q, const float* v, float* o) {
  float uv[3], uuv[3];
  cross3(q, v, uv);
  cross3(q, uv, uuv);
  for (int k = 0; k < 3; ++k) o[k] = v[k] + ((uv[k] * q[3]) + uuv[k]) * 2.0f;
}
// polar observation (rho, -phi) of the goal in the agent's frame (simulator.cpp:666-676)
BPSX_DEV void write_polar(const AgentArrays& A, uint32_t gi, const float* pos, const float* q, const float* goal) {
  const float v[3] = {goal[0] - pos[0], goal[1] - pos[1], goal[2] - pos[2]};
  const float qxx = q[0] * q[0], qyy = q[1] * q[1], qzz = q[2] * q[2];
  const float qxz = q[0] * q[2], qxy = q[0] * q[1], qyz = q[1] * q[2];
  const float qwx = q[3] * q[0], qwy = q[3] * q[1], qwz = q[3] * q[2];
  const float m00 = 1.0f - 2.0f * (qyy + qzz), m01 = 2.0f * (qxy + qwz), m02 = 2.0f * (qxz - qwy);
  const float m20 = 2.0f * (qxz + qwy), m21 = 2.0f * (qyz - qwx), m22 = 1.0f - 2.0f * (qxx + qyy);
  const float vx = m00 * v[0] + m01 * v[1] + m02 * v[2];
  const float vz = m20 * v[0] + m21 * v[1] + m22 * v[2];
  const float x = -vz, y = vx;
  A.polars[(size_t)gi * 2 + 0] = sqrtf(x * x + y * y);
  A.polars[(size_t)gi * 2 + 1] = -atan2f(y, x);
}

// Appends one item per lane with `pred` to a queue: one atomic per wavefront.
BPSX_DEV uint32_t wave_append(bool pred, uint32_t* counter) {
  const unsigned long long m = __ballot(pred);
  if (!m) return 0;
  const int lane = (int)(threadIdx.x & 63);
  const int leader = __ffsll((long long)m) - 1;
  uint32_t base = 0;
  if (lane == leader) base = atomicAdd(counter, (uint32_t)__popcll(m));
  base = (uint32_t)__shfl((int)base, leader);
  return base + (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
}

BPSX_DEV void load3(const float* p, size_t i, float* o) { o[0] = p[i * 3]; o[1] = p[i * 3 + 1]; o[2] = p[i * 3 + 2]; }
BPSX_DEV void store3(float* p, size_t i, const float* v) { p[i * 3] = v[0]; p[i * 3 + 1] = v[1]; p[i * 3 + 2] = v[2]; }

// Exploration::InfoFunctor::update (simulator.cpp:897-904): the cell of the agent in the frame
// of the episode's start pose joins the episode's set.  Returns the set's size.
BPSX_DEV uint32_t visit_cell(const AgentArrays& A, uint32_t gi, const float* pos) {
  float ip[3], iq[4];
  load3(A.exp_init, gi, ip);
  for (int k = 0; k < 4; ++k) iq[k] = A.exp_inv[(size_t)gi * 4 + k];
  const float d[3] = {pos[0] - ip[0], pos[1] - ip[1], pos[2] - ip[2]};
  float g[3];
  quat_rotate(iq, d, g);
  // int(x) of the reference; for a value no int32 holds (or NaN) the x86 conversion the
  // reference compiles to gives INT32_MIN, the GPU's would saturate: made explicit
  auto cell = [](float x) { return (x > -2147483648.0f && x < 2147483648.0f) ? (int32_t)x : (int32_t)0x80000000; };
  const int32_t c0 = cell(g[0] / 1.0f), c1 = cell(g[1] / 1.0f), c2 = cell(g[2] / 1.0f);
  int32_t* cells = A.exp_cells + (size_t)gi * A.cell_cap * 3;
  const uint32_t n = A.exp_count[gi];
  for (uint32_t i = 0; i < n; ++i)
    if (cells[i * 3] == c0 && cells[i * 3 + 1] == c1 && cells[i * 3 + 2] == c2) return n;
  if (n >= A.cell_cap) return n;   // cannot happen: one update per step and per reset
  cells[n * 3] = c0; cells[n * 3 + 1] = c1; cells[n * 3 + 2] = c2;
  A.exp_count[gi] = n + 1;
  return n + 1;
}

// makes scene-table entry `target` what the envs of `slot` move to when their episodes end
__global__ void k_set_swap(uint32_t* swap_target, uint32_t* swap_remaining, uint32_t slot, uint32_t target, uint32_t envs) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    swap_remaining[slot] = envs;
    swap_target[slot] = target;
  }
}

// Empties all of Q, and the reset list and the ticket counters of R (which may be Q again): R's
// lists of queries may already hold what an earlier launch has put there for the coming one.
__global__ void k_clear_queues(StepQueues Q, StepQueues R) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    for (int c = 0; c < kGeoClasses; ++c) Q.counts[kQGeo + c] = 0;
    Q.counts[kQGeoHead] = 0; Q.counts[kQReset] = 0;
    R.counts[kQGeoHead] = 0; R.counts[kQReset] = 0;
  }
}

// Picks the next episode of agent gi and writes its pose; the snaps follow in reset_snap.
BPSX_DEV void begin_reset(const NavData& nav, const AgentArrays& A, const StepParams& P, uint32_t gi) {
  const uint32_t count = A.nresets[gi];
  A.nresets[gi] = count + 1;
  A.step[gi] = 1;
  A.last_cost[gi] = kCostUnknown;
  const uint32_t sc = A.scene[gi];
  const SceneDev& s = nav.scenes[sc];
  const uint64_t key = reset_key(P.seed, gi, count);
  float ep[10];
  if (P.reset_mode == 0) {
    const uint32_t e = draw_index(reset_draw(key, 0), s.ep_count);
    A.episode[gi] = e;
    for (int k = 0; k < 10; ++k) ep[k] = nav.episodes[(size_t)(s.ep_base + e) * 10 + k];
  } else {
    A.episode[gi] = 0;
    float a[3] = {0, 0, 0}, b[3] = {0, 0, 0};
    uint32_t ip;
    sample_point(nav, s, draw_unit(reset_draw(key, 0)), draw_unit(reset_draw(key, 1)), draw_unit(reset_draw(key, 2)), a, &ip);
    sample_point(nav, s, draw_unit(reset_draw(key, 3)), draw_unit(reset_draw(key, 4)), draw_unit(reset_draw(key, 5)), b, &ip);
    const uint32_t turns = draw_index(reset_draw(key, 6), 36);
    float q[4] = {0, 0, 0, 1};
    for (uint32_t t = 0; t < turns; ++t) quat_mul(q, P.turn_left, q);
    ep[0] = a[0]; ep[1] = a[1]; ep[2] = a[2];
    ep[3] = q[0]; ep[4] = q[1]; ep[5] = q[2]; ep[6] = q[3];
    ep[7] = b[0]; ep[8] = b[1]; ep[9] = b[2];
  }
  store3(A.pos, gi, ep);
  for (int k = 0; k < 4; ++k) A.rot[(size_t)gi * 4 + k] = ep[3 + k];
  store3(A.goal, gi, ep + 7);
}

__global__ __launch_bounds__(64) void k_step_move(NavData nav, AgentArrays A, StepQueues Q, StepParams P,
                                                   const int64_t* __restrict__ actions) {
  __shared__ MoveLds move_lds;
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  bool want = false, reset = false;
  uint32_t cls = 0;
  GeoQuery q{};
  uint32_t movePolys = 0, gi = 0;
  if (i < P.n) {
    gi = P.base + i;
    const int64_t action = actions[i];
    if (action < 0 || action > 3) {
      // the reference aborts here (simulator.cpp:704-708); flag it and leave the agent alone
      atomicOr(P.error_flag, 1u);
      A.flags[gi] = kAgentSkip;
    } else {
      // Everything the step may need of the agent is read here, before the first store: the
      // loads then go out together instead of one dependent round trip after the other.
      const uint32_t step = A.step[gi] + 1;
      const uint32_t scene0 = A.scene[gi];
      float pos[3], rot[4], goal[3], navNow[3], goalNav[3];
      load3(A.pos, gi, pos);
      load3(A.goal, gi, goal);
      for (int k = 0; k < 4; ++k) rot[k] = A.rot[(size_t)gi * 4 + k];
      load3(A.nav_xyz, gi, navNow);
      uint32_t navRefNow = A.nav_ref[gi];
      load3(A.goal_xyz, gi, goalNav);
      const uint32_t goalRef = A.goal_ref[gi];
      const bool distOk = A.dist_ok[gi] == 1;
      const uint32_t expected = A.last_cost[gi];
      A.step[gi] = step;
      bool done = (float)step >= P.max_steps;
      bool moved = false;
      // The goal->agent distance is a deterministic function of the two navmesh points. When
      // the agent's point is bit-identical to the one the last step query of this episode was
      // made for (blocked forward move, turn, stop), that query's result is the answer again.
      bool samePoint = true;
      if (action == 0) {
        done = true;
      } else {
        if (action == 1) {
          const float fwd[3] = {0.f * 0.25f, 0.f * 0.25f, -1.f * 0.25f};
          float delta[3];
          quat_rotate(rot, fwd, delta);
          const SceneDev& s = nav.scenes[scene0];
          const NavPt st{navNow[0], navNow[1], navNow[2], navRefNow};
          const NavPt r = try_step(nav, s, st, pos[0] + delta[0], pos[1] + delta[1], pos[2] + delta[2], &movePolys, move_lds);
          samePoint = __float_as_uint(r.x) == __float_as_uint(st.x) && __float_as_uint(r.y) == __float_as_uint(st.y) &&
                      __float_as_uint(r.z) == __float_as_uint(st.z) && r.ref == st.ref;
          pos[0] = r.x; pos[1] = r.y; pos[2] = r.z;
          navNow[0] = r.x; navNow[1] = r.y; navNow[2] = r.z;
          navRefNow = r.ref;
          store3(A.nav_xyz, gi, pos);
          A.nav_ref[gi] = r.ref;
          store3(A.pos, gi, pos);
          moved = true;
        } else {
          quat_mul(rot, action == 2 ? P.turn_left : P.turn_right, rot);
          for (int k = 0; k < 4; ++k) A.rot[(size_t)gi * 4 + k] = rot[k];
        }
        write_polar(A, gi, pos, rot, goal);
      }
      // PointNav measures the distance on every move and at the end of the episode, Flee on
      // moves only, Exploration never (simulator.cpp:758-790, 845-856, 918-927)
      const bool measure = P.task == BPSX_TASK_POINTNAV ? (done || moved) : (P.task == BPSX_TASK_FLEE && moved);
      const bool reuse = measure && samePoint && distOk;
      A.flags[gi] = (done ? kAgentDone : 0u) | (moved ? kAgentMoved : 0u) | (reuse ? kAgentReuse : 0u);
      if (P.task == BPSX_TASK_EXPLORATION) {
        // the count is taken before the pose arrays move on to the next episode
        uint32_t cnt = A.exp_count[gi];
        if (moved) cnt = visit_cell(A, gi, pos);
        A.geo[gi] = (float)(cnt - 1);
      }
      if (measure && !reuse) {
        want = true;
        for (int k = 0; k < 3; ++k) { q.a[k] = goalNav[k]; q.b[k] = navNow[k]; }
        q.a_ref = goalRef;
        q.b_ref = navRefNow;
        q.scene = scene0;
        q.out = gi;
        q.cost_slot = done ? kNoCostSlot : gi;   // a finished episode's search predicts nothing
        q.pad = 0;
        cls = expected == kCostUnknown ? kGeoClassUnknown : geo_class(expected);
      }
      if (done) {
        // the terminal query above holds copies of the old episode's points: the pose arrays can
        // take the next episode now; distance bookkeeping waits for step_finish.  If a new scene
        // waits for this env's slot, the next episode is drawn there (simulator.cpp:1636-1642).
        {
          const uint32_t cur = scene0, tgt = P.swap_target[cur % P.num_slots];
          if (tgt != kNoSwap && tgt != cur) {
            A.scene[gi] = tgt;
            atomicSub(&P.swap_remaining[cur % P.num_slots], 1u);
          }
        }
        begin_reset(nav, A, P, gi);
        reset = true;
      }
    }
  }
  // queue the queries: one atomic per wavefront and class present in it, all of them in flight
  // together (per-lane atomics on the sixteen class counters serialise, and so do the round
  // trips of one atomic per class after the other)
  {
    const int lane = (int)(threadIdx.x & 63);
    unsigned long long mine = 0;   // lanes of this wavefront that queue into the same class as this one
    for (uint32_t c = 0; c < (uint32_t)kGeoClasses; ++c) {
      const unsigned long long m = __ballot(want && cls == c);
      if (want && cls == c) mine = m;
    }
    const int leader = want ? __ffsll((long long)mine) - 1 : lane;
    uint32_t base = 0;
    if (want && lane == leader) base = atomicAdd(&Q.counts[kQGeo + cls], (uint32_t)__popcll(mine));
    base = (uint32_t)__shfl((int)base, leader);
    if (want) Q.queries[(size_t)cls * Q.stride + base + (uint32_t)__popcll(mine & ((1ull << lane) - 1ull))] = q;
  }
  const uint32_t rslot = wave_append(reset, &Q.counts[kQReset]);
  if (reset) Q.reset_list[rslot] = gi;
  // counters, one atomic per wavefront
  const unsigned long long mv = __ballot(movePolys != 0);
  uint32_t mp = movePolys;
  for (int o = 32; o > 0; o >>= 1) mp += (uint32_t)__shfl_xor((int)mp, o);
  if ((threadIdx.x & 63) == 0) {
    if (mv) {
      atomicAdd((unsigned long long*)&P.counters[kCntForward], (unsigned long long)__popcll(mv));
      atomicAdd((unsigned long long*)&P.counters[kCntMovePolys], (unsigned long long)mp);
    }
  }
  if (i == 0) atomicAdd((unsigned long long*)&P.counters[kCntSteps], (unsigned long long)P.n);
}

// served: the counters of the lists of queries that this step's searches have just served;
// before: those of the other set.  Both are left as the next step expects them, so that a step
// needs no launch of its own for it: the served lists and their ticket counter empty, and the
// reset list of the step before empty (its snaps, which read it, ended before this step began).
__global__ __launch_bounds__(256) void k_step_finish(AgentArrays A, StepParams P, uint32_t* served, uint32_t* before) {
  if (blockIdx.x == 0) {
    static_assert(kQGeoHead == kQGeo + kGeoClasses && kGeoClasses + 1 < 256, "one thread per counter");
    if (threadIdx.x <= (uint32_t)kGeoClasses) served[kQGeo + threadIdx.x] = 0;
    else if (threadIdx.x == (uint32_t)kGeoClasses + 1u) before[kQReset] = 0;
  }
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P.n) return;
  const uint32_t gi = P.base + i;
  const uint32_t f = A.flags[gi];
  if (f & kAgentSkip) return;
  const bool done = f & kAgentDone, moved = f & kAgentMoved;
  if (P.task != BPSX_TASK_POINTNAV) {
    if (!(f & kAgentResetOnly)) {
      float v, reward;
      if (P.task == BPSX_TASK_FLEE) {
        v = A.info_prev[gi];
        if (moved) {
          if (!(f & kAgentReuse)) v = A.geo[gi];
          A.info_prev[gi] = v;
          A.dist_ok[gi] = 1;
        }
        reward = v - A.rew_prev[gi];
      } else {
        v = A.geo[gi];
        reward = (float)(0.25 * (double)(v - A.rew_prev[gi]));
      }
      A.rew_prev[gi] = v;
      A.rewards[gi] = reward;
      A.masks[gi] = done ? 0 : 1;
      A.infos[gi] = v;
    }
    if (done || (f & kAgentResetOnly)) {
      // Flee: distance 0 at the start; Exploration: the start cell is in the set (count 1)
      A.info_prev[gi] = 0.0f;
      A.rew_prev[gi] = 0.0f;
      A.dist_ok[gi] = 0;
    }
    return;
  }
  if (A.dist_ok[gi] == 2) {
    // the episode began in the previous step: its first distance has been measured in this one
    const float d = A.geo[(size_t)P.total + gi];
    A.init[gi] = d;
    A.info_prev[gi] = d;   // agent->goal: not a goal->agent result, so not reusable
    A.rew_prev[gi] = d;
    A.dist_ok[gi] = 0;
  }
  if (!(f & kAgentResetOnly)) {
    float dist, success = 0, spl = 0;
    const float fresh = (f & kAgentReuse) ? A.info_prev[gi] : A.geo[gi];
    if (done) {
      dist = fresh;
      success = dist < 0.2f ? 1.0f : 0.0f;
      const float init = A.init[gi], cum = A.cum[gi];
      const float mx = init < cum ? cum : init;
      spl = success * init / mx;
    } else if (moved) {
      dist = fresh;
      A.dist_ok[gi] = 1;
      float pos[3], pp[3];
      load3(A.pos, gi, pos);
      load3(A.prev_pos, gi, pp);
      const float dx = pos[0] - pp[0], dy = pos[1] - pp[1], dz = pos[2] - pp[2];
      A.cum[gi] = A.cum[gi] + sqrtf(dx * dx + dy * dy + dz * dz);
      A.info_prev[gi] = dist;
      store3(A.prev_pos, gi, pos);
    } else {
      dist = A.info_prev[gi];
    }
    float reward = -1e-2f;
    if (done) reward += 2.5f * spl;
    else reward += A.rew_prev[gi] - dist;
    A.rew_prev[gi] = dist;
    A.rewards[gi] = reward;
    A.masks[gi] = done ? 0 : 1;
    A.infos[(size_t)gi * 3 + 0] = success;
    A.infos[(size_t)gi * 3 + 1] = spl;
    A.infos[(size_t)gi * 3 + 2] = dist;
  }
  if (done || (f & kAgentResetOnly)) {
    // InfoFunctor::reset / RewardFunctor::reset with the new episode's first distance, which a
    // step leaves to the next step's launch (no output of this step depends on it)
    A.cum[gi] = 0;
    if (P.defer_first_distance && !(f & kAgentResetOnly)) {
      A.dist_ok[gi] = 2;
    } else {
      const float d = A.geo[(size_t)P.total + gi];
      A.init[gi] = d;
      A.info_prev[gi] = d;   // agent->goal: not a goal->agent result, so not reusable
      A.dist_ok[gi] = 0;
      A.rew_prev[gi] = d;
    }
    float pos[3];
    load3(A.pos, gi, pos);
    store3(A.prev_pos, gi, pos);
  }
}

__global__ __launch_bounds__(256) void k_reset_all(NavData nav, AgentArrays A, StepQueues Q, StepParams P) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= P.n) return;
  const uint32_t gi = P.base + i;
  begin_reset(nav, A, P, gi);
  A.flags[gi] = kAgentResetOnly;
  Q.reset_list[i] = gi;
  if (i == 0) Q.counts[kQReset] = P.n;
}

// One block of two wavefronts per agent being reset: each takes one snap of the new episode (the
// two are independent chains of dependent loads), then the first writes the state, the polar
// observation and the episode's first geodesic query.
__global__ __launch_bounds__(128) void k_reset_snap(NavData nav, AgentArrays A, StepQueues Q, StepQueues Qout, StepParams P) {
  __shared__ SnapLds lds[2];
  __shared__ NavPt goalPt;
  const uint32_t n = Q.counts[kQReset];
  const int lane = (int)(threadIdx.x & 63), half = (int)(threadIdx.x >> 6);
  uint32_t cands = 0;
  for (uint32_t i = blockIdx.x; i < n; i += gridDim.x) {
    const uint32_t gi = Q.reset_list[i];
    const SceneDev& s = nav.scenes[A.scene[gi]];
    float pos[3], goal[3], rot[4];
    load3(A.pos, gi, pos);
    load3(A.goal, gi, goal);
    for (int k = 0; k < 4; ++k) rot[k] = A.rot[(size_t)gi * 4 + k];
    const bool pointnav = P.task == BPSX_TASK_POINTNAV;   // the other tasks snap no goal (simulator.cpp:838-843, 906-916)
    NavPt a{};
    if (half == 0) a = snap_point_wave(nav, s, pos[0], pos[1], pos[2], lds[0], &cands);
    else if (pointnav) {
      const NavPt b = snap_point_wave(nav, s, goal[0], goal[1], goal[2], lds[1], &cands);
      if (lane == 0) goalPt = b;
    }
    __syncthreads();
    if (!pointnav) {
      // no first query either
      if (threadIdx.x == 0) {
        const float axyz[3] = {a.x, a.y, a.z}, zero[3] = {0, 0, 0};
        store3(A.nav_xyz, gi, axyz);
        A.nav_ref[gi] = a.ref;
        const bool flee = P.task == BPSX_TASK_FLEE;
        store3(A.goal_xyz, gi, flee ? axyz : zero);   // Flee: navmeshStart_
        A.goal_ref[gi] = flee ? a.ref : 0u;
        write_polar(A, gi, pos, rot, goal);
        if (!flee) {
          // glm::inverse(q) = conjugate(q) / dot(q, q)
          const float d = (rot[3] * rot[3] + rot[0] * rot[0]) + (rot[1] * rot[1] + rot[2] * rot[2]);
          const float inv[4] = {-rot[0] / d, -rot[1] / d, -rot[2] / d, rot[3] / d};
          for (int k = 0; k < 4; ++k) A.exp_inv[(size_t)gi * 4 + k] = inv[k];
          store3(A.exp_init, gi, pos);
          A.exp_count[gi] = 0;
          visit_cell(A, gi, pos);
        }
      }
    } else if (threadIdx.x == 0) {
      const NavPt b = goalPt;
      const float axyz[3] = {a.x, a.y, a.z}, bxyz[3] = {b.x, b.y, b.z};
      store3(A.nav_xyz, gi, axyz);
      A.nav_ref[gi] = a.ref;
      store3(A.goal_xyz, gi, bxyz);
      A.goal_ref[gi] = b.ref;
      write_polar(A, gi, pos, rot, goal);
      GeoQuery q;
      q.a[0] = a.x; q.a[1] = a.y; q.a[2] = a.z; q.a_ref = a.ref;
      q.b[0] = b.x; q.b[1] = b.y; q.b[2] = b.z; q.b_ref = b.ref;
      q.scene = A.scene[gi];
      q.out = P.total + gi;
      q.cost_slot = kNoCostSlot;   // searched agent -> goal: says little about the searches to come
      q.pad = 0;
      // a new episode: no history
      Qout.queries[(size_t)kGeoClassUnknown * Qout.stride + atomicAdd(&Qout.counts[kQGeo + kGeoClassUnknown], 1u)] = q;
    }
    __syncthreads();   // goalPt is rewritten in the next round
  }
  if (threadIdx.x == 0 && blockIdx.x == 0 && n) atomicAdd((unsigned long long*)&P.counters[kCntResets], (unsigned long long)n);
  if (lane == 0 && cands) atomicAdd((unsigned long long*)&P.counters[kCntSnapCands], (unsigned long long)cands);
}

#ifdef BPSX_QUERY_TRACE
#include "diag_trace.h"   // diagnostic build only: per-query trace buffer
#endif
// Work of one wavefront on one query, whichever instantiation g belongs to: the search, the
// result and the agent's cost estimate.
struct GeoTotals {
  uint32_t pops = 0, corridor = 0, done = 0;
};
template <class Wave>
BPSX_DEV void serve_query(Wave& g, const NavData& nav, const GeoQuery& q, int cls, float* out, uint32_t* last_cost, GeoTotals& T) {
  const uint32_t pops0 = T.pops;
#ifdef BPSX_QUERY_TRACE
  const unsigned long long trace_t0 = wall_clock64();
  const uint32_t trace_replays0 = g.tieReplays, trace_spills0 = g.linkSpills, trace_bridges0 = g.exactRuns;
  const unsigned long long trace_pred = (last_cost && q.cost_slot != kNoCostSlot) ? last_cost[q.cost_slot] : 0xffffu;
#endif
  // the longer the expected search, the sooner its instructions issue; a search of unknown
  // length may be among the longest, but most are not: they run just below those known to be long
  set_wave_priority(cls == (int)kGeoClassUnknown ? 2 : (int)(((uint32_t)(kGeoClasses - 1 - cls) * kGeoClassWidth) / 400u));
  const float d = geodesic_query(g, nav, q, &T.pops, &T.corridor);
  if (g.lane == 0) {
#ifdef BPSX_QUERY_TRACE
    const unsigned int ti = atomicAdd(&g_trace_n, 1u);
    if (ti < (1u << 17)) {
      g_trace[ti][0] = trace_t0; g_trace[ti][1] = wall_clock64(); g_trace[ti][2] = T.pops - pops0;
      // class, predicted length, ties resolved from the log, link spills, bridges to the exact loops
      g_trace[ti][3] = (unsigned long long)cls | ((trace_pred & 0xffffu) << 8) | ((unsigned long long)((g.tieReplays - trace_replays0) & 0xfffu) << 24) |
                        ((unsigned long long)((g.linkSpills - trace_spills0) & 0xfffu) << 36) | ((unsigned long long)((g.exactRuns - trace_bridges0) & 0xffu) << 48);
    }
#endif
    out[q.out] = d;
    // estimate for the agent's next search: this one's length, decaying from earlier peaks
    if (last_cost && q.cost_slot != kNoCostSlot) {
      const uint32_t prev = last_cost[q.cost_slot], now = T.pops - pops0;
      const uint32_t faded = prev == kCostUnknown ? 0u : prev - (prev >> 2);
      last_cost[q.cost_slot] = now > faded ? now : faded;
    }
  }
  T.done++;
  wave_sync();
}

// Blocks of two wavefronts, each wavefront persistent and serving queries from the shared
// queue on its half of the block's LDS.  The launch ends with its longest search, so the
// queries of the kLongClasses longest classes are treated apart: block b takes the b-th of
// them, if there is one, and gives it the whole block's LDS (the larger instantiation: no link
// spills, half the window misses, shorter hash chains; 7 % faster on such searches) while its
// second wavefront leaves.  Every other wavefront's first query is fixed by its index too;
// from the second query on a wavefront draws from the queue's counter.
constexpr int kLongClasses = (int)geo_class(1400);   // the classes of an expected cost of 1400 nodes and more
__global__ __launch_bounds__(128) __attribute__((amdgpu_waves_per_eu(5, 5))) void k_geodesic(NavData nav, const GeoQuery* __restrict__ queries, uint32_t stride,
                                                  const uint32_t* __restrict__ counts, uint32_t* head,
                                                  float* out, uint32_t* last_cost, GeoSlot* slots, uint64_t* counters) {
  constexpr size_t kHalf = sizeof(geo::GeoShared);
  static_assert(kHalf % 16 == 0 && sizeof(geo_long::GeoShared) <= 2 * kHalf, "the long search must fit the LDS of one block");
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * kHalf];
  const int lane = (int)(threadIdx.x & 63), half = uniform_i((int)(threadIdx.x >> 6));   // the same in all lanes, and known to be: addresses derived from it stay in scalar registers
  GeoSlot* slot = &slots[blockIdx.x * 2 + half];
  // Classes are served in order: class c owns the ticket numbers from the sum of the counts
  // before it.  A wavefront's tickets only go up, so it keeps the class it is in and that
  // class's range of tickets, and moves on through the counts as its tickets pass the range.
  uint32_t nq = 0, nlong = 0;
  for (int c = 0; c < kGeoClasses; ++c) {
    nq += (uint32_t)uniform_i((int)counts[c]);
    if (c + 1 == kLongClasses) nlong = nq;
  }
  int curCls = 0;
  uint32_t curLo = 0, curHi = (uint32_t)uniform_i((int)counts[0]);
  auto class_of = [&](uint32_t ticket) {   // ticket < nq, not below an earlier one
    while (ticket >= curHi) {
      curCls++;
      curLo = curHi;
      curHi += (uint32_t)uniform_i((int)counts[curCls]);
    }
    return curCls;
  };
  GeoTotals T;
  uint32_t linkSpills = 0, heapSpills = 0, exactRuns = 0, tieReplays = 0, pairTies = 0;
  // The first query of every wavefront needs no ticket counter: the grid is what the device
  // holds at once, so block b takes long query b if there is one, and the wavefronts of the
  // other blocks take the queries after the long ones in the order of their index.  (Some
  // thousand atomics on one counter at the start of a launch are served one after the other.)
  const uint32_t lt = blockIdx.x;
  if (lt < nlong) {
    if (half == 1) return;
    geo_long::GeoWave gl;
    gl.lane = lane;
    gl.L = &reinterpret_cast<geo_long::GeoShared*>(lds)->a;
    gl.ws = slot;
    gl.heapSize = 0;
    gl.nodeCount = 0;
    gl.linkSpills = gl.heapSpills = gl.exactRuns = gl.tieReplays = gl.pairTies = 0;
#ifdef BPSX_PHASE_TIMING
    for (int k = 0; k < 8; ++k) gl.phase[k] = 0;
#endif
    const int cls = class_of(lt);
    const GeoQuery q = queries[(size_t)cls * stride + (lt - curLo)];
    serve_query(gl, nav, q, cls, out, last_cost, T);
    linkSpills += gl.linkSpills; heapSpills += gl.heapSpills; exactRuns += gl.exactRuns; tieReplays += gl.tieReplays; pairTies += gl.pairTies;
    if (lane == 0) atomicAdd((unsigned long long*)&counters[kCntLongPath], 1ull);
#ifdef BPSX_PHASE_TIMING
    if (lane == 0) for (int k = 0; k < 8; ++k) atomicAdd((unsigned long long*)&counters[8 + k], gl.phase[k]);
#endif
  }
  geo::GeoWave g;
  g.lane = lane;
  g.L = &reinterpret_cast<geo::GeoShared*>(lds + (size_t)half * kHalf)->a;
  g.ws = slot;
  g.heapSize = 0;
  g.nodeCount = 0;
  g.linkSpills = g.heapSpills = g.exactRuns = g.tieReplays = g.pairTies = 0;
#ifdef BPSX_PHASE_TIMING
  for (int k = 0; k < 8; ++k) g.phase[k] = 0;
#endif
  // tickets below `taken` went to the blocks' first wavefronts above
  const uint32_t taken = nlong < gridDim.x ? nlong : gridDim.x;
  const uint32_t nstatic = (gridDim.x - taken) * 2u;   // wavefronts that start on the general queries
  bool firstQuery = blockIdx.x >= taken;
  for (;;) {
    uint32_t qi = 0;
    if (firstQuery) {
      qi = taken + (blockIdx.x - taken) * 2u + (uint32_t)half;
      firstQuery = false;
    } else {
      if (lane == 0) qi = atomicAdd(head, 1u);
      qi = taken + nstatic + (uint32_t)uniform_i((int)qi);
    }
    if (qi >= nq) break;
    const int cls = class_of(qi);
    const GeoQuery q = queries[(size_t)cls * stride + (qi - curLo)];
    serve_query(g, nav, q, cls, out, last_cost, T);
  }
  linkSpills += g.linkSpills; heapSpills += g.heapSpills; exactRuns += g.exactRuns; tieReplays += g.tieReplays; pairTies += g.pairTies;
  if (lane == 0 && T.done) {
    atomicAdd((unsigned long long*)&counters[kCntGeoQueries], (unsigned long long)T.done);
    atomicAdd((unsigned long long*)&counters[kCntAstarPops], (unsigned long long)T.pops);
    atomicAdd((unsigned long long*)&counters[kCntCorridor], (unsigned long long)T.corridor);
    if (linkSpills) atomicAdd((unsigned long long*)&counters[kCntLinkSpills], (unsigned long long)linkSpills);
    if (heapSpills) atomicAdd((unsigned long long*)&counters[kCntHeapSpills], (unsigned long long)heapSpills);
    if (exactRuns) atomicAdd((unsigned long long*)&counters[kCntExactRuns], (unsigned long long)exactRuns);
    if (tieReplays) atomicAdd((unsigned long long*)&counters[kCntTieReplays], (unsigned long long)tieReplays);
    if (pairTies) atomicAdd((unsigned long long*)&counters[kCntPairTies], (unsigned long long)pairTies);
#ifdef BPSX_PHASE_TIMING
    for (int k = 0; k < 8; ++k) atomicAdd((unsigned long long*)&counters[8 + k], g.phase[k]);
#endif
  }
}

// ---- batched PathFinder-level kernels (one lane per item, or one group per item)
__global__ __launch_bounds__(64) void k_snap_batch(NavData nav, uint32_t scene, const float* pts, uint32_t n, float* oxyz,
                                                   uint32_t* oref) {
  __shared__ SnapLds lds;
  uint32_t c = 0;
  for (uint32_t i = blockIdx.x; i < n; i += gridDim.x) {
    const NavPt r = snap_point_wave(nav, nav.scenes[scene], pts[(size_t)i * 3], pts[(size_t)i * 3 + 1], pts[(size_t)i * 3 + 2], lds, &c);
    if (threadIdx.x == 0) {
      oxyz[(size_t)i * 3] = r.x; oxyz[(size_t)i * 3 + 1] = r.y; oxyz[(size_t)i * 3 + 2] = r.z;
      oref[i] = r.ref;
    }
  }
}
__global__ void k_try_step_batch(NavData nav, uint32_t scene, const float* sxyz, const uint32_t* sref, const float* exyz,
                                 uint32_t n, float* oxyz, uint32_t* oref) {
  __shared__ MoveLds move_lds;
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  uint32_t c = 0;
  NavPt st{sxyz[(size_t)i * 3], sxyz[(size_t)i * 3 + 1], sxyz[(size_t)i * 3 + 2], sref[i]};
  const NavPt r = try_step(nav, nav.scenes[scene], st, exyz[(size_t)i * 3], exyz[(size_t)i * 3 + 1], exyz[(size_t)i * 3 + 2], &c, move_lds);
  oxyz[(size_t)i * 3] = r.x; oxyz[(size_t)i * 3 + 1] = r.y; oxyz[(size_t)i * 3 + 2] = r.z;
  oref[i] = r.ref;
}
__global__ void k_make_queries(uint32_t scene, const float* sxyz, const uint32_t* sref, const float* exyz,
                               const uint32_t* eref, uint32_t n, GeoQuery* q) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  GeoQuery o;
  for (int k = 0; k < 3; ++k) { o.a[k] = sxyz[(size_t)i * 3 + k]; o.b[k] = exyz[(size_t)i * 3 + k]; }
  o.a_ref = sref[i]; o.b_ref = eref[i]; o.scene = scene; o.out = i;
  o.cost_slot = kNoCostSlot; o.pad = 0;
  q[i] = o;
}
__global__ void k_random_points(NavData nav, uint32_t scene, const float* u, uint32_t n, float* oxyz, uint32_t* oref) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const SceneDev& s = nav.scenes[scene];
  float p[3] = {0, 0, 0};
  uint32_t ip = 0;
  const bool ok = sample_point(nav, s, u[(size_t)i * 3], u[(size_t)i * 3 + 1], u[(size_t)i * 3 + 2], p, &ip);
  oxyz[(size_t)i * 3] = p[0]; oxyz[(size_t)i * 3 + 1] = p[1]; oxyz[(size_t)i * 3 + 2] = p[2];
  oref[i] = ok ? (s.ref_base | ip) : 0;
}
// counts and both ticket counters of a batch of n queries, all in the class of the shortest
__global__ void k_set_counts(uint32_t* p, uint32_t n) {
  if (threadIdx.x <= (uint32_t)kGeoClasses) p[threadIdx.x] = threadIdx.x == (uint32_t)kGeoClasses - 1u ? n : 0u;
}

}  // namespace

// ------------------------------------------------------------------ launch wrappers
static inline dim3 grid_for(uint32_t n, uint32_t block) { return dim3((n + block - 1) / block); }

uint32_t geodesic_blocks_per_cu() {
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, k_geodesic, 128, 0) != hipSuccess || n < 1) n = 1;
  return (uint32_t)n;
}

// num_blocks blocks of two wavefronts; slots holds one GeoSlot per wavefront
void launch_geodesic(const NavData& nav, const GeoQuery* queries, uint32_t stride, const uint32_t* counts, uint32_t* head,
                     float* out, uint32_t* last_cost, GeoSlot* slots, uint32_t num_blocks,
                     uint64_t* counters, hipStream_t st) {
  hipLaunchKernelGGL(k_geodesic, dim3(num_blocks), dim3(128), 0, st, nav, queries, stride, counts, head, out,
                     last_cost, slots, counters);
}

void launch_step(const NavData& nav, const AgentArrays& A, const StepQueues& Q, const StepQueues& Qnext, const StepParams& P,
                 const int64_t* actions_dev, GeoSlot* slots, uint32_t geo_blocks, uint32_t snap_blocks, hipStream_t st,
                 hipStream_t side, hipEvent_t moved, hipEvent_t snapped, hipEvent_t* ev) {
  int e = 0;
  auto mark = [&]() { if (ev) (void)hipEventRecord(ev[e++], st); };
  mark();
  // Q's lists of queries were emptied two steps ago and have since taken the first queries of
  // the episodes that began in the previous step; its reset list and ticket counter, and the
  // lists of Qnext, were emptied by the previous step's last launch
  hipLaunchKernelGGL(k_step_move, grid_for(P.n, 64), dim3(64), 0, st, nav, A, Q, P, actions_dev);
  mark();
  // the new episodes' snaps need nothing of this step's searches and the searches nothing of
  // them: they run side by side
  // (not when the launches are being timed one by one: then everything stays on st)
  const bool fork = side && !ev;
  if (fork) {
    (void)hipEventRecord(moved, st);
    (void)hipStreamWaitEvent(side, moved, 0);
  }
  // (a grid for one agent in sixteen ending its episode; more take further rounds.  Blocks
  // without work would only wait for LDS that the searches hold and keep the join waiting.)
  const uint32_t step_snap_blocks = std::min(snap_blocks, std::max(64u, P.n / 16u));
  hipLaunchKernelGGL(k_reset_snap, dim3(step_snap_blocks), dim3(128), 0, fork ? side : st, nav, A, Q, Qnext, P);
  if (fork) (void)hipEventRecord(snapped, side);
  mark();
  launch_geodesic(nav, Q.queries, Q.stride, &Q.counts[kQGeo], &Q.counts[kQGeoHead], A.geo,
                  A.last_cost, slots, geo_blocks, P.counters, st);
  mark();
  hipLaunchKernelGGL(k_step_finish, grid_for(P.n, 256), dim3(256), 0, st, A, P, Q.counts, Qnext.counts);
  if (fork) (void)hipStreamWaitEvent(st, snapped, 0);
  mark();
}

void launch_reset(const NavData& nav, const AgentArrays& A, const StepQueues& Q, const StepQueues& Qother, const StepParams& P,
                  GeoSlot* slots, uint32_t geo_blocks, uint32_t snap_blocks, hipStream_t st) {
  hipLaunchKernelGGL(k_clear_queues, dim3(1), dim3(64), 0, st, Q, Qother);
  hipLaunchKernelGGL(k_clear_queues, dim3(1), dim3(64), 0, st, Qother, Qother);
  hipLaunchKernelGGL(k_reset_all, grid_for(P.n, 256), dim3(256), 0, st, nav, A, Q, P);
  hipLaunchKernelGGL(k_reset_snap, dim3(snap_blocks), dim3(128), 0, st, nav, A, Q, Q, P);
  launch_geodesic(nav, Q.queries, Q.stride, &Q.counts[kQGeo], &Q.counts[kQGeoHead], A.geo,
                  A.last_cost, slots, geo_blocks, P.counters, st);
  hipLaunchKernelGGL(k_step_finish, grid_for(P.n, 256), dim3(256), 0, st, A, P, Q.counts, Qother.counts);
  // the next step finds its lists of queries empty, not with this launch's queries still in them
  hipLaunchKernelGGL(k_clear_queues, dim3(1), dim3(64), 0, st, Q, Q);
}

void launch_snap_batch(const NavData& nav, uint32_t scene, const float* pts, uint32_t n, float* oxyz, uint32_t* oref,
                       uint32_t snap_blocks, hipStream_t st) {
  hipLaunchKernelGGL(k_snap_batch, dim3(snap_blocks < n ? snap_blocks : n), dim3(64), 0, st, nav, scene, pts, n, oxyz, oref);
}
void launch_try_step_batch(const NavData& nav, uint32_t scene, const float* sxyz, const uint32_t* sref, const float* exyz,
                           uint32_t n, float* oxyz, uint32_t* oref, hipStream_t st) {
  hipLaunchKernelGGL(k_try_step_batch, grid_for(n, 64), dim3(64), 0, st, nav, scene, sxyz, sref, exyz, n, oxyz, oref);
}
void launch_geodesic_batch(const NavData& nav, uint32_t scene, const float* sxyz, const uint32_t* sref, const float* exyz,
                           const uint32_t* eref, uint32_t n, GeoQuery* qbuf, uint32_t* count_head /* [kGeoClasses + 1] */, float* out,
                           GeoSlot* slots, uint32_t geo_blocks, uint64_t* counters, hipStream_t st) {
  hipLaunchKernelGGL(k_make_queries, grid_for(n, 256), dim3(256), 0, st, scene, sxyz, sref, exyz, eref, n, qbuf);
  hipLaunchKernelGGL(k_set_counts, dim3(1), dim3(128), 0, st, count_head, n);
  // one class only: stride 0 puts its queries at the start of the buffer
  launch_geodesic(nav, qbuf, 0, &count_head[0], &count_head[kGeoClasses], out, nullptr, slots,
                  geo_blocks, counters, st);
}
void launch_set_swap(uint32_t* swap_target, uint32_t* swap_remaining, uint32_t slot, uint32_t target, uint32_t envs,
                     hipStream_t st) {
  hipLaunchKernelGGL(k_set_swap, dim3(1), dim3(64), 0, st, swap_target, swap_remaining, slot, target, envs);
}
void launch_random_points(const NavData& nav, uint32_t scene, const float* u, uint32_t n, float* oxyz, uint32_t* oref,
                          hipStream_t st) {
  hipLaunchKernelGGL(k_random_points, grid_for(n, 64), dim3(64), 0, st, nav, scene, u, n, oxyz, oref);
}

#ifdef BPSX_QUERY_TRACE
#define BPSX_DIAG_TRACE_HOST
#include "diag_trace.h"
#endif
}  // namespace bpsx
