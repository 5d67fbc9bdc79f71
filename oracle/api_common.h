// TEST INFRASTRUCTURE — the extern "C" surface shared by liboracle.so (independent
// restatement) and oracle/_ref/libbpsref.so (compiled reference PathFinder): identical
// symbol names so that tests drive either through one ctypes wrapper.
#pragma once
#include <cstdint>
#include <cstring>
#include <string>

#include "sim_core.h"

#define BPO_API extern "C" __attribute__((visibility("default")))

template <class B>
struct ApiImpl {
  using SimT = simcore::Sim<B>;

  struct Nav {
    std::vector<std::shared_ptr<typename B::Scene>> scenes;
    std::unique_ptr<typename B::Ctx> ctx;
  };

  static std::string& err() {
    static thread_local std::string e;
    return e;
  }

  static void* nav_load(const void* bytes, size_t n) {
    auto s = B::load((const uint8_t*)bytes, n, &err());
    if (!s) return nullptr;
    Nav* nav = new Nav();
    nav->scenes.push_back(s);
    nav->ctx = B::make_ctx(nav->scenes);
    return nav;
  }
  static void nav_snap(void* h, const float* pts, uint32_t n, float* oxyz, uint32_t* oref) {
    Nav* nav = (Nav*)h;
    for (uint32_t i = 0; i < n; ++i) {
      const simcore::NavPt r = nav->ctx->snap(0, &pts[(size_t)i * 3]);
      memcpy(&oxyz[(size_t)i * 3], r.xyz, 12);
      oref[i] = r.ref;
    }
  }
  static void nav_try_step(void* h, const float* sxyz, const uint32_t* sref, const float* exyz, uint32_t n,
                           float* oxyz, uint32_t* oref) {
    Nav* nav = (Nav*)h;
    for (uint32_t i = 0; i < n; ++i) {
      simcore::NavPt s;
      memcpy(s.xyz, &sxyz[(size_t)i * 3], 12);
      s.ref = sref[i];
      const simcore::NavPt r = nav->ctx->tryStep(0, s, &exyz[(size_t)i * 3]);
      memcpy(&oxyz[(size_t)i * 3], r.xyz, 12);
      oref[i] = r.ref;
    }
  }
  static void nav_geodesic(void* h, const float* sxyz, const uint32_t* sref, const float* exyz,
                           const uint32_t* eref, uint32_t n, float* out) {
    Nav* nav = (Nav*)h;
    for (uint32_t i = 0; i < n; ++i) {
      simcore::NavPt a, b;
      memcpy(a.xyz, &sxyz[(size_t)i * 3], 12); a.ref = sref[i];
      memcpy(b.xyz, &exyz[(size_t)i * 3], 12); b.ref = eref[i];
      out[i] = nav->ctx->geodesic(0, a, b);
    }
  }
  static void nav_sample(void* h, const float* u, uint32_t n, float* oxyz) {
    Nav* nav = (Nav*)h;
    for (uint32_t i = 0; i < n; ++i)
      nav->ctx->sample(0, u[(size_t)i * 3], u[(size_t)i * 3 + 1], u[(size_t)i * 3 + 2], &oxyz[(size_t)i * 3]);
  }
  static void nav_free(void* h) { delete (Nav*)h; }

  static void* sim_create(uint32_t numEnvs, uint32_t numScenes, uint32_t doubleBuffered, uint32_t resetMode,
                          uint64_t seed, uint32_t maxSteps, int numThreads) {
    return new SimT(numEnvs, numScenes, doubleBuffered != 0, resetMode, seed, maxSteps, numThreads);
  }
  static int sim_add_scene(void* h, const void* bytes, size_t n, const float* episodes, uint32_t E) {
    return ((SimT*)h)->addScene((const uint8_t*)bytes, n, episodes, E, &err()) ? 0 : -1;
  }
  static int sim_finalize(void* h) { return ((SimT*)h)->finalize(&err()) ? 0 : -1; }
  static void sim_get_outputs(void* h, uint32_t g, float* rewards, uint8_t* masks, float* infos, float* polars) {
    SimT* s = (SimT*)h;
    const uint32_t n = s->envsPerGroup();
    memcpy(rewards, s->rewards(g), (size_t)n * 4);
    memcpy(masks, s->masks(g), n);
    memcpy(infos, s->infos(g), (size_t)n * 12);
    memcpy(polars, s->polars(g), (size_t)n * 8);
  }
  static void sim_get_state(void* h, uint32_t g, float* pos, float* rot, float* goal, uint32_t* poly,
                            uint32_t* goalRef, uint32_t* step, uint32_t* episode, uint32_t* numResets) {
    SimT* s = (SimT*)h;
    const uint32_t n = s->envsPerGroup();
    for (uint32_t i = 0; i < n; ++i) {
      const simcore::Env& e = s->env(g, i);
      memcpy(&pos[(size_t)i * 3], e.pos, 12);
      memcpy(&rot[(size_t)i * 4], e.rot, 16);
      memcpy(&goal[(size_t)i * 3], e.goal, 12);
      poly[i] = e.nav.ref;
      goalRef[i] = e.navGoal.ref;
      step[i] = e.step;
      episode[i] = e.episode;
      numResets[i] = e.numResets;
    }
  }
};

#define BPO_DEFINE_API(B)                                                                                   \
  BPO_API const char* bpo_last_error() { return ApiImpl<B>::err().c_str(); }                                \
  BPO_API void* bpo_nav_load(const void* b, size_t n) { return ApiImpl<B>::nav_load(b, n); }               \
  BPO_API void bpo_nav_snap(void* h, const float* p, uint32_t n, float* ox, uint32_t* orf) {               \
    ApiImpl<B>::nav_snap(h, p, n, ox, orf);                                                                 \
  }                                                                                                         \
  BPO_API void bpo_nav_try_step(void* h, const float* s, const uint32_t* sr, const float* e, uint32_t n,   \
                                float* ox, uint32_t* orf) {                                                 \
    ApiImpl<B>::nav_try_step(h, s, sr, e, n, ox, orf);                                                      \
  }                                                                                                         \
  BPO_API void bpo_nav_geodesic(void* h, const float* s, const uint32_t* sr, const float* e,               \
                                const uint32_t* er, uint32_t n, float* o) {                                 \
    ApiImpl<B>::nav_geodesic(h, s, sr, e, er, n, o);                                                        \
  }                                                                                                         \
  BPO_API void bpo_nav_sample(void* h, const float* u, uint32_t n, float* ox) {                             \
    ApiImpl<B>::nav_sample(h, u, n, ox);                                                                    \
  }                                                                                                         \
  BPO_API void bpo_nav_free(void* h) { ApiImpl<B>::nav_free(h); }                                           \
  BPO_API void* bpo_sim_create(uint32_t ne, uint32_t ns, uint32_t db, uint32_t rm, uint64_t seed,          \
                               uint32_t ms, int nt) {                                                       \
    return ApiImpl<B>::sim_create(ne, ns, db, rm, seed, ms, nt);                                            \
  }                                                                                                         \
  BPO_API int bpo_sim_add_scene(void* h, const void* b, size_t n, const float* ep, uint32_t E) {           \
    return ApiImpl<B>::sim_add_scene(h, b, n, ep, E);                                                       \
  }                                                                                                         \
  BPO_API void bpo_sim_set_task(void* h, uint32_t task) { ((ApiImpl<B>::SimT*)h)->setTask(task); }         \
  BPO_API int bpo_sim_finalize(void* h) { return ApiImpl<B>::sim_finalize(h); }                             \
  BPO_API int bpo_sim_swap_scene(void* h, uint32_t slot, const void* b, size_t n, const float* ep, uint32_t E) { \
    return ((ApiImpl<B>::SimT*)h)->swapScene(slot, (const uint8_t*)b, n, ep, E, &ApiImpl<B>::err()) ? 0 : -1; \
  }                                                                                                         \
  BPO_API uint32_t bpo_sim_swap_remaining(void* h, uint32_t slot) {                                        \
    return ((ApiImpl<B>::SimT*)h)->swapRemaining(slot);                                                     \
  }                                                                                                         \
  BPO_API uint32_t bpo_sim_envs_per_group(void* h) { return ((ApiImpl<B>::SimT*)h)->envsPerGroup(); }      \
  BPO_API void bpo_sim_reset(void* h, uint32_t g) { ((ApiImpl<B>::SimT*)h)->reset(g); }                    \
  BPO_API void bpo_sim_step(void* h, uint32_t g, const int64_t* a) { ((ApiImpl<B>::SimT*)h)->step(g, a); } \
  BPO_API int bpo_sim_bad_action(void* h) { return ((ApiImpl<B>::SimT*)h)->sawBadAction() ? 1 : 0; }       \
  BPO_API void bpo_sim_get_outputs(void* h, uint32_t g, float* r, uint8_t* m, float* i, float* p) {        \
    ApiImpl<B>::sim_get_outputs(h, g, r, m, i, p);                                                          \
  }                                                                                                         \
  BPO_API void bpo_sim_get_state(void* h, uint32_t g, float* pos, float* rot, float* goal, uint32_t* poly, \
                                 uint32_t* gr, uint32_t* st, uint32_t* ep, uint32_t* nr) {                  \
    ApiImpl<B>::sim_get_state(h, g, pos, rot, goal, poly, gr, st, ep, nr);                                  \
  }                                                                                                         \
  BPO_API void bpo_sim_destroy(void* h) { delete (ApiImpl<B>::SimT*)h; }
