// TEST INFRASTRUCTURE — liboracle.so: the independent CPU restatement (nav_oracle +
// sim_core) behind the bpo_* C surface. Loaded only by tests/, smoke() and the
// cpu_baseline leg of bench.py.
#include "api_common.h"
#include "nav_oracle.h"

namespace {

struct OracleBackend {
  struct Scene {
    orc::Mesh* mesh = nullptr;
    ~Scene() { orc::mesh_free(mesh); }
  };
  struct Ctx {
    std::vector<std::unique_ptr<orc::Query>> q;
    static orc::NavPoint in(const simcore::NavPt& p) {
      orc::NavPoint o;
      memcpy(o.xyz, p.xyz, 12);
      o.ref = p.ref;
      return o;
    }
    static simcore::NavPt out(const orc::NavPoint& p) {
      simcore::NavPt o;
      memcpy(o.xyz, p.xyz, 12);
      o.ref = p.ref;
      return o;
    }
    simcore::NavPt snap(uint32_t s, const float* p) { return out(q[s]->snapPoint(p)); }
    simcore::NavPt tryStep(uint32_t s, const simcore::NavPt& a, const float* end) { return out(q[s]->tryStep(in(a), end)); }
    float geodesic(uint32_t s, const simcore::NavPt& a, const simcore::NavPt& b) { return q[s]->geodesic(in(a), in(b)); }
    bool sample(uint32_t s, float u0, float sv, float tv, float* xyz) {
      uint32_t ref;
      return q[s]->samplePoint(u0, sv, tv, xyz, &ref);
    }
  };
  static std::shared_ptr<Scene> load(const uint8_t* b, size_t n, std::string* err) {
    orc::Mesh* m = orc::mesh_load(b, n, err);
    if (!m) return nullptr;
    auto s = std::make_shared<Scene>();
    s->mesh = m;
    return s;
  }
  static std::unique_ptr<Ctx> make_ctx(const std::vector<std::shared_ptr<Scene>>& scenes) {
    auto c = std::make_unique<Ctx>();
    for (auto& s : scenes) c->q.push_back(std::make_unique<orc::Query>(s->mesh));
    return c;
  }
};

}  // namespace

BPO_DEFINE_API(OracleBackend)

BPO_API const char* bpo_kind() { return "port"; }

// Work counters summed over all threads of a simulator: 13 u64 in the order of orc::Counters.
BPO_API void bpo_sim_counters(void* h, uint64_t* out) {
  auto* s = (ApiImpl<OracleBackend>::SimT*)h;
  orc::Counters total;
  for (int t = 0; t < s->numThreads(); ++t)
    for (auto& q : s->ctx(t).q) total.add(q->counters);
  const uint64_t v[13] = {total.move_calls, total.move_polys, total.move_verts, total.height_tris, total.path_calls,
                          total.astar_pops, total.astar_links, total.corridor_polys, total.snap_calls,
                          total.snap_bv_nodes, total.snap_cands, total.snap_cand_verts, total.snap_cand_tris};
  memcpy(out, v, sizeof(v));
}

// Mesh introspection for tests.
BPO_API int bpo_nav_poly_count(void* h) {
  return orc::mesh_poly_count(((ApiImpl<OracleBackend>::Nav*)h)->scenes[0]->mesh);
}
BPO_API void bpo_nav_poly_info(void* h, uint32_t* refs, uint16_t* flags, int32_t* islands) {
  const orc::Mesh* m = ((ApiImpl<OracleBackend>::Nav*)h)->scenes[0]->mesh;
  const int n = orc::mesh_poly_count(m);
  for (int i = 0; i < n; ++i) {
    refs[i] = orc::mesh_poly_ref(m, i);
    flags[i] = orc::mesh_poly_flags(m, i);
    islands[i] = orc::mesh_poly_island(m, i);
  }
}
// Corridor (polygon refs) of the last geodesic query that reached the funnel.
BPO_API int bpo_nav_last_corridor(void* h, uint32_t* out, int max) {
  const auto& c = ((ApiImpl<OracleBackend>::Nav*)h)->ctx->q[0]->lastCorridor();
  const int n = (int)c.size() < max ? (int)c.size() : max;
  memcpy(out, c.data(), (size_t)n * 4);
  return (int)c.size();
}
// Distances of the goal-rooted distance-field formulation (orc::Query::geodesicViaField), for
// the measurement of how far that formulation is from the reference's findPath.
BPO_API void bpo_nav_geodesic_field(void* h, const float* sxyz, const uint32_t* sref, const float* exyz,
                                    const uint32_t* eref, uint32_t n, float* out) {
  orc::Query& q = *((ApiImpl<OracleBackend>::Nav*)h)->ctx->q[0];
  for (uint32_t i = 0; i < n; ++i) {
    orc::NavPoint a, b;
    memcpy(a.xyz, &sxyz[(size_t)i * 3], 12); a.ref = sref[i];
    memcpy(b.xyz, &exyz[(size_t)i * 3], 12); b.ref = eref[i];
    out[i] = q.geodesicViaField(a, b);
  }
}
// Switches the check of the multi-node pass rules on (rows 1..4) or off (0) for the scene's
// query object and returns its counts so far: passes, nodes, wrongNode, wrongUpdate, pairs, ties.
BPO_API void bpo_nav_pass_check(void* h, int rows, uint64_t* out) {
  orc::Query& q = *((ApiImpl<OracleBackend>::Nav*)h)->ctx->q[0];
  const orc::Query::PassCheck& p = q.passCheck;
  out[0] = p.passes; out[1] = p.nodes; out[2] = p.wrongNode; out[3] = p.wrongUpdate; out[4] = p.pairs; out[5] = p.ties;
  q.passCheck = orc::Query::PassCheck();
  q.passCheck.rows = rows;
}
BPO_API void bpo_random_point_in_convex_poly(const float* pts, int npts, float s, float t, float* out) {
  float areas[16];
  orc::random_point_in_convex_poly(pts, npts, areas, s, t, out);
}
