// TEST INFRASTRUCTURE — oracle/_ref/libbpsref.so: the reference's own PathFinder + Detour,
// compiled from the sources where they lie under /root/reference, behind the same bpo_* C
// surface as liboracle.so.  Only this adapter is repository code; no reference source is
// copied.  PathFinder loads from a file path (PathFinder.cpp:330), so blobs go through a
// temporary file.  Each thread context owns a full set of PathFinders, as each reference
// worker thread does (simulator.cpp:1712-1730).
#include <unistd.h>

#include <cstdio>
#include <cstdlib>

#include "DetourCommon.h"
#include "DetourNavMesh.h"
#include "DetourNavMeshQuery.h"
#include "PathFinder.h"
#include "api_common.h"

namespace {

struct RefBackend {
  struct Scene {
    std::string path;  // temporary .navmesh file
    std::vector<uint8_t> bytes;
    ~Scene() { if (!path.empty()) unlink(path.c_str()); }
  };
  // A second, directly driven Detour mesh per scene for the sampled-reset spec (the
  // PathFinder pimpl hides its dtNavMesh).
  struct RawMesh {
    dtNavMesh* mesh = nullptr;
    dtNavMeshQuery* query = nullptr;
    std::vector<float> areaCum;
    std::vector<dtPolyRef> refs;
    ~RawMesh() { dtFreeNavMeshQuery(query); dtFreeNavMesh(mesh); }
  };
  struct Ctx {
    std::vector<std::unique_ptr<esp::nav::PathFinder>> pf;
    std::vector<std::unique_ptr<RawMesh>> raw;
    static esp::nav::NavMeshPoint in(const simcore::NavPt& p) {
      esp::nav::NavMeshPoint o;
      o.xyz = esp::vec3f(p.xyz[0], p.xyz[1], p.xyz[2]);
      o.polyId = p.ref;
      return o;
    }
    static simcore::NavPt out(const esp::nav::NavMeshPoint& p) {
      simcore::NavPt o;
      o.xyz[0] = p.xyz[0]; o.xyz[1] = p.xyz[1]; o.xyz[2] = p.xyz[2];
      o.ref = (uint32_t)p.polyId;
      return o;
    }
    simcore::NavPt snap(uint32_t s, const float* p) { return out(pf[s]->snapPoint(esp::vec3f(p[0], p[1], p[2]))); }
    simcore::NavPt tryStep(uint32_t s, const simcore::NavPt& a, const float* e) {
      return out(pf[s]->tryStep(in(a), esp::vec3f(e[0], e[1], e[2])));
    }
    float geodesic(uint32_t s, const simcore::NavPt& a, const simcore::NavPt& b) {
      path_.requestedStart = in(a);
      path_.requestedEnd = in(b);
      pf[s]->findPath(path_);
      return path_.geodesicDistance;
    }
    // The engine's sampling rule evaluated with the reference's own dtTriArea2D,
    // dtRandomPointInConvexPoly and getPolyHeight.
    bool sample(uint32_t s, float u0, float sv, float tv, float* xyz) {
      RawMesh& r = *raw[s];
      const int n = (int)r.areaCum.size();
      const float total = n ? r.areaCum[n - 1] : 0.0f;
      if (!(total > 0.0f)) return false;
      const float target = u0 * total;
      int lo = 0, hi = n - 1;
      while (lo < hi) {
        const int mid = (lo + hi) / 2;
        if (r.areaCum[mid] > target) hi = mid;
        else lo = mid + 1;
      }
      const dtMeshTile* tile = 0;
      const dtPoly* poly = 0;
      r.mesh->getTileAndPolyByRefUnsafe(r.refs[lo], &tile, &poly);
      float verts[3 * DT_VERTS_PER_POLYGON], areas[DT_VERTS_PER_POLYGON];
      for (int j = 0; j < poly->vertCount; ++j) dtVcopy(&verts[j * 3], &tile->verts[poly->verts[j] * 3]);
      float pt[3];
      dtRandomPointInConvexPoly(verts, poly->vertCount, areas, sv, tv, pt);
      float h = 0;
      if (dtStatusSucceed(r.query->getPolyHeight(r.refs[lo], pt, &h))) pt[1] = h;
      dtVcopy(xyz, pt);
      return true;
    }
    esp::nav::ShortestPath path_;
  };

  static std::shared_ptr<Scene> load(const uint8_t* b, size_t n, std::string* err) {
    char tmpl[] = "/tmp/bpsref_XXXXXX";
    const int fd = mkstemp(tmpl);
    if (fd < 0) { *err = "mkstemp failed"; return nullptr; }
    FILE* fp = fdopen(fd, "wb");
    fwrite(b, 1, n, fp);
    fclose(fp);
    auto s = std::make_shared<Scene>();
    s->path = tmpl;
    s->bytes.assign(b, b + n);
    esp::nav::PathFinder probe;
    if (!probe.loadNavMesh(s->path)) { *err = "PathFinder::loadNavMesh failed"; return nullptr; }
    return s;
  }
  static std::unique_ptr<RawMesh> load_raw(const Scene& s) {
    // same steps as PathFinder::loadNavMesh, on the in-memory bytes
    auto r = std::make_unique<RawMesh>();
    const uint8_t* b = s.bytes.data();
    dtNavMeshParams params;
    int numTiles;
    memcpy(&numTiles, b + 8, 4);
    memcpy(&params, b + 12, sizeof(params));
    r->mesh = dtAllocNavMesh();
    r->mesh->init(&params);
    size_t off = 40;
    for (int i = 0; i < numTiles; ++i) {
      dtTileRef ref; int size;
      memcpy(&ref, b + off, 4); memcpy(&size, b + off + 4, 4);
      off += 8;
      if (!ref || !size) break;
      unsigned char* data = (unsigned char*)dtAlloc(size, DT_ALLOC_PERM);
      memcpy(data, b + off, size);
      off += size;
      r->mesh->addTile(data, size, DT_TILE_FREE_DATA, ref, 0);
    }
    r->query = dtAllocNavMeshQuery();
    r->query->init(r->mesh, 2048);
    float acc = 0.0f;
    const dtNavMesh* cm = r->mesh;
    for (int it = 0; it < cm->getMaxTiles(); ++it) {
      const dtMeshTile* tile = cm->getTile(it);
      if (!tile || !tile->header) continue;
      const dtPolyRef base = cm->getPolyRefBase(tile);
      for (int i = 0; i < tile->header->polyCount; ++i) {
        const dtPoly* p = &tile->polys[i];
        // zero-area polygons are disabled by PathFinder (PathFinder.cpp:307-328); none of
        // the meshes used with sampled resets contain any, so flags are taken as stored
        if (p->getType() == DT_POLYTYPE_GROUND && (p->flags & 0x01)) {
          float a = 0.0f;
          for (int j = 2; j < p->vertCount; ++j)
            a += dtTriArea2D(&tile->verts[p->verts[0] * 3], &tile->verts[p->verts[j - 1] * 3], &tile->verts[p->verts[j] * 3]);
          if (a > 0.0f) acc += a;
        }
        r->areaCum.push_back(acc);
        r->refs.push_back(base | (dtPolyRef)i);
      }
    }
    return r;
  }
  static std::unique_ptr<Ctx> make_ctx(const std::vector<std::shared_ptr<Scene>>& scenes) {
    auto c = std::make_unique<Ctx>();
    for (auto& s : scenes) {
      auto pf = std::make_unique<esp::nav::PathFinder>();
      if (!pf->loadNavMesh(s->path)) abort();
      c->pf.push_back(std::move(pf));
      c->raw.push_back(load_raw(*s));
    }
    return c;
  }
};

float g_frand_state_u[1];
uint64_t g_frand_s;
float frand_stream() {
  g_frand_s = simcore::mix64(g_frand_s + 0x9E3779B97F4A7C15ull);
  return (float)(g_frand_s >> 40) * (1.0f / 16777216.0f);
}

}  // namespace

BPO_DEFINE_API(RefBackend)

BPO_API const char* bpo_kind() { return "reference"; }

// dtNavMeshQuery::findRandomPoint driven by a seeded stream, for distribution checks.
BPO_API void bpo_nav_find_random_points(void* h, uint64_t seed, uint32_t n, float* oxyz, uint32_t* oref) {
  auto* nav = (ApiImpl<RefBackend>::Nav*)h;
  RefBackend::RawMesh& r = *nav->ctx->raw[0];
  dtQueryFilter filter;
  filter.setIncludeFlags(0x01);
  filter.setExcludeFlags(0);
  g_frand_s = seed;
  for (uint32_t i = 0; i < n; ++i) {
    dtPolyRef ref = 0;
    float pt[3] = {0, 0, 0};
    r.query->findRandomPoint(&filter, frand_stream, &ref, pt);
    memcpy(&oxyz[(size_t)i * 3], pt, 12);
    oref[i] = ref;
  }
}
BPO_API void bpo_random_point_in_convex_poly(const float* pts, int npts, float s, float t, float* out) {
  float areas[16];
  dtRandomPointInConvexPoly(pts, npts, areas, s, t, out);
}
// dtCreateNavMeshData on a caller-described polygon soup, for packer byte-parity checks.
#include "DetourNavMeshBuilder.h"
BPO_API int bpo_ref_create_tile(const uint16_t* verts, int vertCount, const uint16_t* polys, const uint16_t* flags,
                                const uint8_t* areas, int polyCount, int nvp, float wh, float wr, float wc,
                                const float* bmin, const float* bmax, float cs, float ch, uint8_t* out, int outCap) {
  dtNavMeshCreateParams p;
  memset(&p, 0, sizeof(p));
  p.verts = verts; p.vertCount = vertCount;
  p.polys = polys; p.polyFlags = flags; p.polyAreas = areas; p.polyCount = polyCount; p.nvp = nvp;
  p.walkableHeight = wh; p.walkableRadius = wr; p.walkableClimb = wc;
  dtVcopy(p.bmin, bmin); dtVcopy(p.bmax, bmax);
  p.cs = cs; p.ch = ch; p.buildBvTree = true;
  unsigned char* data = 0;
  int size = 0;
  if (!dtCreateNavMeshData(&p, &data, &size)) return -1;
  if (size <= outCap) memcpy(out, data, size);
  dtFree(data);
  return size;
}
