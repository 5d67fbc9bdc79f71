// Navmesh upload, host half.  Does what PathFinder::loadNavMesh does before the first query
// (PathFinder.cpp:330-408): read the MSET container, place the tile (dtNavMesh::init/addTile,
// DetourNavMesh.cpp:224-265, 908-1048), disable zero-area polygons (:276-328), label connected
// components (IslandSystem :53-170) — and writes the result as flat arrays for the GPU
// instead of Detour's pointer-linked tile.  Only single-tile meshes are accepted.
#include "navmesh_host.h"

#include <cmath>
#include <cstring>
#include <initializer_list>

#include "../../include/bpsx.h"
#include "dt_format.h"
#include "errors.h"

namespace bpsx {

int parse_navmesh(const uint8_t* b, size_t n, HostScene* out) {
  if (!b || !out) return fail(BPSX_E_INVAL, "navmesh: null argument");
  if (n < sizeof(MsetHeader)) return fail(BPSX_E_INVAL, "navmesh: truncated MSET header");
  MsetHeader mh;
  memcpy(&mh, b, sizeof(mh));
  if (mh.magic != kMsetMagic) return fail(BPSX_E_INVAL, "navmesh: bad MSET magic");
  if (mh.version != kMsetVersion) return fail(BPSX_E_INVAL, "navmesh: bad MSET version");
  if (mh.params.maxTiles < 1 || mh.params.maxPolys < 1) return fail(BPSX_E_INVAL, "navmesh: bad params");
  const uint32_t tileBits = ilog2(nextPow2((uint32_t)mh.params.maxTiles));
  const uint32_t polyBits = ilog2(nextPow2((uint32_t)mh.params.maxPolys));
  if (tileBits + polyBits > 22) return fail(BPSX_E_INVAL, "navmesh: params leave fewer than 10 salt bits");
  const uint32_t saltBits = std::min(31u, 32 - tileBits - polyBits);

  size_t off = sizeof(MsetHeader);
  const uint8_t* tileData = nullptr;
  MsetTileHeader th{};
  int tiles = 0;
  for (int t = 0; t < mh.numTiles; ++t) {
    if (off + sizeof(MsetTileHeader) > n) return fail(BPSX_E_INVAL, "navmesh: truncated tile header");
    MsetTileHeader cur;
    memcpy(&cur, b + off, sizeof(cur));
    off += sizeof(cur);
    if (!cur.tileRef || !cur.dataSize) break;
    if (cur.dataSize < (int)sizeof(TileHeader) || off + (size_t)cur.dataSize > n)
      return fail(BPSX_E_INVAL, "navmesh: truncated tile data");
    if (tiles == 0) { tileData = b + off; th = cur; }
    tiles++;
    off += (size_t)cur.dataSize;
  }
  if (tiles == 0) return fail(BPSX_E_INVAL, "navmesh: holds no tile");
  // The reference cannot load these either: PathFinder builds polygon refs with salt and tile
  // index swapped (PathFinder.cpp:67, 318), which only cancels out for a one-tile mesh.
  if (tiles > 1) return fail(BPSX_E_UNSUPPORTED, "navmesh: multi-tile meshes are not supported (nor by the reference's PathFinder)");

  TileHeader h;
  memcpy(&h, tileData, sizeof(h));
  if (h.magic != kTileMagic) return fail(BPSX_E_INVAL, "navmesh: bad tile magic");
  if (h.version != kTileVersion) return fail(BPSX_E_INVAL, "navmesh: bad tile version");
  if (h.offMeshConCount != 0) return fail(BPSX_E_UNSUPPORTED, "navmesh: off-mesh connections are not supported");
  if (h.polyCount < 1 || h.polyCount > 0x7fff || h.vertCount < 1 || h.detailMeshCount != h.polyCount ||
      h.maxLinkCount < 0 || h.detailVertCount < 0 || h.detailTriCount < 0 || h.bvNodeCount < 0)
    return fail(BPSX_E_INVAL, "navmesh: inconsistent tile header");
  if ((uint32_t)h.polyCount > (1u << polyBits)) return fail(BPSX_E_INVAL, "navmesh: polyCount exceeds maxPolys bits");
  // the device tree names its right children and leaves in 16 bits, 0xffff marks a leaf
  if (h.bvNodeCount > 0xfffe) return fail(BPSX_E_INVAL, "navmesh: more BV nodes than a tile of 32767 polygons can have");
  // no section can hold more elements than the tile has bytes: checked before the counts are
  // multiplied, and the sizes are computed in size_t
  const size_t tileBytes = (size_t)th.dataSize;
  for (const int count : {h.vertCount, h.polyCount, h.maxLinkCount, h.detailMeshCount, h.detailVertCount, h.detailTriCount,
                          h.bvNodeCount})
    if ((size_t)count > tileBytes) return fail(BPSX_E_INVAL, "navmesh: a section count exceeds the tile size");
  const size_t headerSize = align4(sizeof(TileHeader));
  const size_t vertsSize = align4((size_t)12 * (size_t)h.vertCount);
  const size_t polysSize = align4((size_t)32 * (size_t)h.polyCount);
  const size_t linksSize = align4((size_t)12 * (size_t)h.maxLinkCount);
  const size_t dmSize = align4((size_t)12 * (size_t)h.detailMeshCount);
  const size_t dvSize = align4((size_t)12 * (size_t)h.detailVertCount);
  const size_t dtSize = align4((size_t)4 * (size_t)h.detailTriCount);
  const size_t bvSize = align4((size_t)16 * (size_t)h.bvNodeCount);
  if (headerSize + vertsSize + polysSize + linksSize + dmSize + dvSize + dtSize + bvSize > (size_t)th.dataSize)
    return fail(BPSX_E_INVAL, "navmesh: tile sections exceed tile size");
  const float* verts = reinterpret_cast<const float*>(tileData + headerSize);
  const uint8_t* pp = tileData + headerSize + vertsSize;
  const uint8_t* dm = pp + polysSize + linksSize;
  const uint8_t* dv = dm + dmSize;
  const uint8_t* dt = dv + dvSize;
  const uint8_t* bvp = dt + dtSize;

  const uint32_t tileIndex = (th.tileRef >> polyBits) & ((1u << tileBits) - 1);
  const uint32_t salt = (th.tileRef >> (polyBits + tileBits)) & ((1u << saltBits) - 1);
  if (tileIndex >= (uint32_t)mh.params.maxTiles) return fail(BPSX_E_INVAL, "navmesh: tile index out of range");

  HostScene& s = *out;
  const int np = h.polyCount;
  s.polys.assign((size_t)np, PolyRec{});
  s.dverts.assign((const float*)dv, (const float*)dv + (size_t)h.detailVertCount * 3);
  s.dtris.assign(dt, dt + (size_t)h.detailTriCount * 4);
  std::vector<TilePoly> tp((size_t)np);
  memcpy(tp.data(), pp, (size_t)np * sizeof(TilePoly));
  std::vector<TilePolyDetail> td((size_t)np);
  memcpy(td.data(), dm, (size_t)np * sizeof(TilePolyDetail));

  for (int i = 0; i < np; ++i) {
    const TilePoly& p = tp[i];
    PolyRec& r = s.polys[i];
    if (p.vertCount < 3 || p.vertCount > kNvp) return fail(BPSX_E_INVAL, "navmesh: polygon vertex count out of range");
    r.nv = p.vertCount;
    r.type = p.areaAndType >> 6;
    if (r.type != 0) return fail(BPSX_E_UNSUPPORTED, "navmesh: off-mesh polygons are not supported");
    r.flags = p.flags;
    for (int k = 0; k < p.vertCount; ++k) {
      if (p.verts[k] >= h.vertCount) return fail(BPSX_E_INVAL, "navmesh: vertex index out of range");
      memcpy(r.v[k], &verts[(size_t)p.verts[k] * 3], 12);
      r.nei[k] = p.neis[k];
      if (p.neis[k] && !(p.neis[k] & kExtLink) && p.neis[k] - 1 >= np)
        return fail(BPSX_E_INVAL, "navmesh: neighbour index out of range");
    }
    const TilePolyDetail& d = td[i];
    if ((size_t)d.triBase + d.triCount > (size_t)h.detailTriCount ||
        (size_t)d.vertBase + d.vertCount > (size_t)h.detailVertCount)
      return fail(BPSX_E_INVAL, "navmesh: detail mesh out of range");
    for (int j = 0; j < d.triCount; ++j)
      for (int k = 0; k < 3; ++k)
        if (s.dtris[(size_t)(d.triBase + j) * 4 + k] >= p.vertCount + d.vertCount)
          return fail(BPSX_E_INVAL, "navmesh: detail triangle vertex out of range");
    r.tri_base = d.triBase;
    r.dvert_base = d.vertBase;
    r.tri_count = d.triCount;
    r.dvert_count = d.vertCount;
  }

  // removeZeroAreaPolys: 3-D area of the detail triangles, accumulated the way the
  // reference's mixed float/double expression does.
  for (int i = 0; i < np; ++i) {
    PolyRec& r = s.polys[i];
    float area = 0;
    for (int j = 0; j < r.tri_count; ++j) {
      const uint8_t* t = &s.dtris[(size_t)(r.tri_base + j) * 4];
      const float* v[3];
      for (int k = 0; k < 3; ++k)
        v[k] = t[k] < r.nv ? r.v[t[k]] : &s.dverts[(size_t)(r.dvert_base + (t[k] - r.nv)) * 3];
      float w1[3], w2[3];
      for (int k = 0; k < 3; ++k) { w1[k] = v[1][k] - v[0][k]; w2[k] = v[2][k] - v[0][k]; }
      const float cx = w1[1] * w2[2] - w1[2] * w2[1];
      const float cy = w1[2] * w2[0] - w1[0] * w2[2];
      const float cz = w1[0] * w2[1] - w1[1] * w2[0];
      const float norm = sqrtf(cx * cx + (cy * cy + cz * cz));
      area = (float)((double)area + 0.5 * (double)norm);
    }
    if ((double)area < 1e-5) r.flags = kPolyFlagDisabled;
  }
  // neighbours that pass the query filter (include WALK, exclude nothing)
  for (int i = 0; i < np; ++i) {
    PolyRec& r = s.polys[i];
    for (int k = 0; k < r.nv; ++k) {
      const uint16_t ne = r.nei[k];
      r.walk[k] = (ne && !(ne & kExtLink) && (s.polys[ne - 1].flags & kPolyFlagWalk)) ? ne : 0;
    }
  }
  // per-edge records of the path search
  s.aedges.assign((size_t)np * kEdgeStride, AEdge{{0, 0, 0}, kNoNb});
  for (int i = 0; i < np; ++i) {
    const PolyRec& r = s.polys[i];
    for (int k = 0; k < r.nv; ++k) {
      AEdge& e = s.aedges[(size_t)i * kEdgeStride + k];
      const float* l = r.v[k];
      const float* rt = r.v[(k + 1) % r.nv];
      for (int c = 0; c < 3; ++c) e.mid[c] = (l[c] + rt[c]) * 0.5f;
      e.nb = r.walk[k] ? (uint32_t)(r.walk[k] - 1) : kNoNb;
      // a polygon behind two edges: expanding through the second never changes its node (same
      // position, not a lower cost), so only the first edge leads there
      for (int j = 0; j < k; ++j)
        if (r.walk[j] == r.walk[k]) e.nb = kNoNb;
    }
  }
  // connected components: polygons are seeded in index order, the seed is not filter-checked,
  // neighbours are entered in ascending edge order and popped last-in first-out
  {
    std::vector<int> isl((size_t)np, -1), stack;
    int next = 0;
    for (int sd = 0; sd < np; ++sd) {
      if (isl[sd] >= 0) continue;
      const int id = next++;
      isl[sd] = id;
      stack.push_back(sd);
      while (!stack.empty()) {
        const int ip = stack.back();
        stack.pop_back();
        const PolyRec& r = s.polys[ip];
        for (int k = 0; k < r.nv; ++k) {
          if (!r.walk[k]) continue;
          const int nb = r.walk[k] - 1;
          if (isl[nb] >= 0) continue;
          isl[nb] = id;
          stack.push_back(nb);
        }
      }
    }
    for (int i = 0; i < np; ++i) s.polys[i].island = (uint32_t)isl[i];
  }
  // prefix sums of the fan areas that findRandomPoint weighs polygons by
  float acc = 0.0f;
  for (int i = 0; i < np; ++i) {
    PolyRec& r = s.polys[i];
    if (r.type == 0 && (r.flags & kPolyFlagWalk)) {
      float a = 0.0f;
      for (int j = 2; j < r.nv; ++j) {
        const float abx = r.v[j - 1][0] - r.v[0][0], abz = r.v[j - 1][2] - r.v[0][2];
        const float acx = r.v[j][0] - r.v[0][0], acz = r.v[j][2] - r.v[0][2];
        a += acx * abz - abx * acz;
      }
      if (a > 0.0f) acc += a;
    }
    r.area_cum = acc;
  }

  // BV tree: repack dtBVNode (bounds + int) into BVNodeDev.  Leaves must name valid polygons;
  // an internal node at i with escape e owns nodes (i, i+e): its left child is i+1 and its
  // right child follows the left subtree.  The links are verified so that the kernels'
  // descent always moves to larger indices inside the array.
  s.bv.assign((size_t)h.bvNodeCount, BVNodeDev{});
  bool tree_ok = h.bvNodeCount > 0;
  {
    std::vector<TileBVNode> raw((size_t)h.bvNodeCount);
    if (h.bvNodeCount) memcpy(raw.data(), bvp, (size_t)h.bvNodeCount * sizeof(TileBVNode));
    const int64_t cnt = h.bvNodeCount;
    auto size_of = [&](int64_t i) -> int64_t { return raw[(size_t)i].i >= 0 ? 1 : -(int64_t)raw[(size_t)i].i; };
    for (int64_t i = 0; i < cnt; ++i) {
      const TileBVNode& r = raw[(size_t)i];
      BVNodeDev& o = s.bv[(size_t)i];
      memcpy(o.bmin, r.bmin, 6);
      memcpy(o.bmax, r.bmax, 6);
      if (r.i >= 0) {
        if (r.i >= np) return fail(BPSX_E_INVAL, "navmesh: BV leaf out of range");
        o.a = (uint16_t)r.i;
        o.b = kBVLeaf;
      } else {
        const int64_t e = -(int64_t)r.i;
        if (e < 1 || e > 0xfffe) return fail(BPSX_E_INVAL, "navmesh: BV escape offset out of range");
        o.a = (uint16_t)e;
        const int64_t left = i + 1;
        const int64_t right = left < cnt ? left + size_of(left) : cnt;
        if (left >= cnt || right >= cnt || right >= i + e || right + size_of(right) != i + e) {
          tree_ok = false;
          o.b = (uint16_t)(left < cnt ? left : 0);
        } else {
          o.b = (uint16_t)right;
        }
      }
    }
    // the builder reserves 2N nodes and uses 2N-1: the rest are zero leaves outside the tree;
    // the in-order walk visits them, so the descent must too (they are appended to its frontier)
    if (tree_ok) {
      const int64_t root_size = size_of(0);
      if (root_size > cnt) tree_ok = false;
    }
  }

  SceneDev& d = s.dev;
  d.poly_count = (uint32_t)np;
  d.bv_count = (uint32_t)h.bvNodeCount;
  d.ref_base = (salt << (polyBits + tileBits)) | (tileIndex << polyBits);
  d.poly_mask = (1u << polyBits) - 1;
  memcpy(d.orig, mh.params.orig, 12);
  d.tile_w = mh.params.tileWidth;
  d.tile_h = mh.params.tileHeight;
  d.tx = h.x;
  d.ty = h.y;
  memcpy(d.bmin, h.bmin, 12);
  memcpy(d.bmax, h.bmax, 12);
  d.qfac = h.bvQuantFactor;
  d.climb = h.walkableClimb;
  d.area_total = acc;
  d.bv_tree_ok = tree_ok ? 1u : 0u;
  return BPSX_OK;
}

}  // namespace bpsx
