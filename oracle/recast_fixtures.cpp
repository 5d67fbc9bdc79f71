// TEST INFRASTRUCTURE — builds the Recast-made navmesh fixtures under tests/golden/.
//
// Links the reference's own Recast and Detour sources where they lie (see the Makefile's
// `recast` target); nothing of this runs on the GPU box, only its outputs (".navmesh" files in
// the MSET container that PathFinder::loadNavMesh reads, PathFinder.cpp:330-408) are committed.
// Unlike the grid generator of the product library these meshes have what real habitat
// navmeshes have: irregular polygons from contour simplification, detail meshes with extra
// height samples, eroded borders, islands on top of obstacles, and (second fixture) two floors
// that overlap in xz joined by a ramp.
//
//   recast_fixtures <output directory>
//
// Build parameters follow the benchmark's description of its first configuration: agent radius
// 0.18 m, height 0.88 m, cell 0.05 m, max step 0.2 m; the remaining rcConfig values are the
// customary ones of a solo-mesh build (edge length 12 m, simplification error 1.3, regions of
// at least 8x8 cells merged below 20x20, 6 vertices per polygon, detail sampling 6 cells / 1 cell).
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "DetourNavMesh.h"
#include "DetourNavMeshBuilder.h"
#include "Recast.h"

namespace {

struct Soup {
  std::vector<float> v;
  std::vector<int> t;
  int vert(float x, float y, float z) {
    v.push_back(x); v.push_back(y); v.push_back(z);
    return (int)v.size() / 3 - 1;
  }
  void tri(int a, int b, int c) { t.push_back(a); t.push_back(b); t.push_back(c); }
  // quad given in an order whose first triangle faces up when it is a floor: (x0,z0) (x0,z1) (x1,z1) (x1,z0)
  void quad(int a, int b, int c, int d) { tri(a, b, c); tri(a, c, d); }
  void box(float x0, float y0, float z0, float x1, float y1, float z1) {
    const int p[8] = {vert(x0, y0, z0), vert(x0, y0, z1), vert(x1, y0, z1), vert(x1, y0, z0),
                      vert(x0, y1, z0), vert(x0, y1, z1), vert(x1, y1, z1), vert(x1, y1, z0)};
    quad(p[4], p[5], p[6], p[7]);   // top, facing up
    quad(p[0], p[3], p[2], p[1]);   // bottom
    quad(p[0], p[1], p[5], p[4]);
    quad(p[1], p[2], p[6], p[5]);
    quad(p[2], p[3], p[7], p[6]);
    quad(p[3], p[0], p[4], p[7]);
  }
  void floor(float x0, float z0, float x1, float z1, float y) {
    quad(vert(x0, y, z0), vert(x0, y, z1), vert(x1, y, z1), vert(x1, y, z0));
  }
};

struct Lcg {
  uint64_t s;
  double next() {
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return (double)(s >> 11) / 9007199254740992.0;
  }
  float range(float a, float b) { return a + (float)next() * (b - a); }
};

bool build(const Soup& soup, const std::string& path) {
  rcContext ctx(false);
  rcConfig cfg;
  memset(&cfg, 0, sizeof(cfg));
  cfg.cs = 0.05f;
  cfg.ch = 0.05f;
  cfg.walkableSlopeAngle = 45.0f;
  cfg.walkableHeight = (int)ceilf(0.88f / cfg.ch);
  cfg.walkableClimb = (int)floorf(0.2f / cfg.ch);
  cfg.walkableRadius = (int)ceilf(0.18f / cfg.cs);
  cfg.maxEdgeLen = (int)(12.0f / cfg.cs);
  cfg.maxSimplificationError = 1.3f;
  cfg.minRegionArea = 8 * 8;
  cfg.mergeRegionArea = 20 * 20;
  cfg.maxVertsPerPoly = 6;
  cfg.detailSampleDist = 6.0f * cfg.cs;
  cfg.detailSampleMaxError = 1.0f * cfg.ch;
  const int nv = (int)soup.v.size() / 3, nt = (int)soup.t.size() / 3;
  rcCalcBounds(soup.v.data(), nv, cfg.bmin, cfg.bmax);
  rcCalcGridSize(cfg.bmin, cfg.bmax, cfg.cs, &cfg.width, &cfg.height);

  rcHeightfield* solid = rcAllocHeightfield();
  if (!rcCreateHeightfield(&ctx, *solid, cfg.width, cfg.height, cfg.bmin, cfg.bmax, cfg.cs, cfg.ch)) return false;
  std::vector<unsigned char> areas((size_t)nt, 0);
  rcMarkWalkableTriangles(&ctx, cfg.walkableSlopeAngle, soup.v.data(), nv, soup.t.data(), nt, areas.data());
  if (!rcRasterizeTriangles(&ctx, soup.v.data(), nv, soup.t.data(), areas.data(), nt, *solid, cfg.walkableClimb)) return false;
  rcFilterLowHangingWalkableObstacles(&ctx, cfg.walkableClimb, *solid);
  rcFilterLedgeSpans(&ctx, cfg.walkableHeight, cfg.walkableClimb, *solid);
  rcFilterWalkableLowHeightSpans(&ctx, cfg.walkableHeight, *solid);
  rcCompactHeightfield* chf = rcAllocCompactHeightfield();
  if (!rcBuildCompactHeightfield(&ctx, cfg.walkableHeight, cfg.walkableClimb, *solid, *chf)) return false;
  rcFreeHeightField(solid);
  if (!rcErodeWalkableArea(&ctx, cfg.walkableRadius, *chf)) return false;
  if (!rcBuildDistanceField(&ctx, *chf)) return false;
  if (!rcBuildRegions(&ctx, *chf, 0, cfg.minRegionArea, cfg.mergeRegionArea)) return false;
  rcContourSet* cset = rcAllocContourSet();
  if (!rcBuildContours(&ctx, *chf, cfg.maxSimplificationError, cfg.maxEdgeLen, *cset)) return false;
  rcPolyMesh* pmesh = rcAllocPolyMesh();
  if (!rcBuildPolyMesh(&ctx, *cset, cfg.maxVertsPerPoly, *pmesh)) return false;
  rcPolyMeshDetail* dmesh = rcAllocPolyMeshDetail();
  if (!rcBuildPolyMeshDetail(&ctx, *pmesh, *chf, cfg.detailSampleDist, cfg.detailSampleMaxError, *dmesh)) return false;
  rcFreeCompactHeightfield(chf);
  rcFreeContourSet(cset);

  // every polygon walkable, ground area: what PathFinder's query filter includes (PathFinder.cpp:239-243)
  for (int i = 0; i < pmesh->npolys; ++i) {
    pmesh->areas[i] = 0;
    pmesh->flags[i] = 1;
  }
  dtNavMeshCreateParams p;
  memset(&p, 0, sizeof(p));
  p.verts = pmesh->verts;
  p.vertCount = pmesh->nverts;
  p.polys = pmesh->polys;
  p.polyAreas = pmesh->areas;
  p.polyFlags = pmesh->flags;
  p.polyCount = pmesh->npolys;
  p.nvp = pmesh->nvp;
  p.detailMeshes = dmesh->meshes;
  p.detailVerts = dmesh->verts;
  p.detailVertsCount = dmesh->nverts;
  p.detailTris = dmesh->tris;
  p.detailTriCount = dmesh->ntris;
  p.walkableHeight = 0.88f;
  p.walkableRadius = 0.18f;
  p.walkableClimb = 0.2f;
  memcpy(p.bmin, pmesh->bmin, 12);
  memcpy(p.bmax, pmesh->bmax, 12);
  p.cs = cfg.cs;
  p.ch = cfg.ch;
  p.buildBvTree = true;
  unsigned char* data = nullptr;
  int size = 0;
  if (!dtCreateNavMeshData(&p, &data, &size)) return false;
  int extraVerts = dmesh->nverts, polys = pmesh->npolys;
  for (int i = 0; i < pmesh->npolys; ++i) {
    int n = 0;
    for (int k = 0; k < pmesh->nvp; ++k) n += pmesh->polys[i * 2 * pmesh->nvp + k] != RC_MESH_NULL_IDX;
    extraVerts -= n;
  }
  rcFreePolyMesh(pmesh);
  rcFreePolyMeshDetail(dmesh);

  // a solo mesh saved the way PathFinder::saveNavMesh does (PathFinder.cpp:410-450)
  dtNavMesh* nav = dtAllocNavMesh();
  if (dtStatusFailed(nav->init(data, size, DT_TILE_FREE_DATA))) return false;
  struct { int magic, version, numTiles; dtNavMeshParams params; } header;
  header.magic = 'M' << 24 | 'S' << 16 | 'E' << 8 | 'T';
  header.version = 1;
  header.numTiles = 1;
  memcpy(&header.params, nav->getParams(), sizeof(dtNavMeshParams));
  const dtNavMesh* cnav = nav;
  const dtMeshTile* tile = cnav->getTile(0);
  struct { dtTileRef tileRef; int dataSize; } th;
  th.tileRef = nav->getTileRef(tile);
  th.dataSize = tile->dataSize;
  FILE* f = fopen(path.c_str(), "wb");
  if (!f) return false;
  fwrite(&header, sizeof(header), 1, f);
  fwrite(&th, sizeof(th), 1, f);
  fwrite(tile->data, (size_t)tile->dataSize, 1, f);
  fclose(f);
  printf("%s: %d polygons, %d detail-only vertices, %d bytes\n", path.c_str(), polys, extraVerts, tile->dataSize);
  dtFreeNavMesh(nav);
  return true;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc < 2) {
    fprintf(stderr, "usage: recast_fixtures <output directory>\n");
    return 2;
  }
  const std::string out = argv[1];
  {
    // 10 m x 10 m floor, 8 boxes of side 0.5-2 m: the first benchmark configuration's scene
    Soup s;
    s.floor(0, 0, 10, 10, 0);
    Lcg r{1001};
    for (int i = 0; i < 8; ++i) {
      const float w = r.range(0.5f, 2.0f), d = r.range(0.5f, 2.0f);
      const float x = r.range(0.3f, 9.7f - w), z = r.range(0.3f, 9.7f - d);
      s.box(x, 0, z, x + w, 1.0f, z + d);
    }
    if (!build(s, out + "/recast_room.navmesh")) return 1;
  }
  {
    // two floors that overlap in xz, joined by a ramp; an uneven patch on the lower floor gives
    // the detail mesh height samples of its own
    Soup s;
    s.floor(0, 0, 12, 8, 0);
    s.box(6, 2.4f, 0, 12, 2.6f, 8);                                   // upper floor slab, top at 2.6
    {
      // ramp from (1, 0) up to (6, 2.6) along x, 2 m wide, with side walls below it
      const int a = s.vert(1, 0, 5.5f), b = s.vert(1, 0, 7.5f), c = s.vert(6, 2.6f, 7.5f), d = s.vert(6, 2.6f, 5.5f);
      s.quad(a, b, c, d);
    }
    {
      // a shallow mound on the lower floor: four sloped faces around a raised square
      const float y = 0.3f;
      const int o[4] = {s.vert(2, 0, 1), s.vert(2, 0, 4), s.vert(5, 0, 4), s.vert(5, 0, 1)};
      const int i[4] = {s.vert(3, y, 2), s.vert(3, y, 3), s.vert(4, y, 3), s.vert(4, y, 2)};
      s.quad(i[0], i[1], i[2], i[3]);
      s.quad(o[0], o[1], i[1], i[0]);
      s.quad(o[1], o[2], i[2], i[1]);
      s.quad(o[2], o[3], i[3], i[2]);
      s.quad(o[3], o[0], i[0], i[3]);
    }
    s.box(8, 0, 3, 9, 1.0f, 4.5f);                                    // an obstacle under the upper floor
    s.box(9, 2.6f, 5, 10.5f, 3.6f, 6);                                // and one on it
    if (!build(s, out + "/recast_two_floors.navmesh")) return 1;
  }
  return 0;
}
