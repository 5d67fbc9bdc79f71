// Host-side navmesh producer: Detour tile packer, MSET container writer and the
// synthetic floor-plan generator used for benchmark and test inputs.
//
// The packer writes the byte layout that dtCreateNavMeshData produces
// (DetourNavMeshBuilder.cpp:280-658; bounding-volume tree :171-241) so that the blobs
// load unchanged in habitat-sim's PathFinder::loadNavMesh (PathFinder.cpp:330-408).
// Off-mesh connections and externally supplied detail meshes are not produced: the
// height mesh is the polygon fan, as the reference builder emits when no detail mesh
// is given (DetourNavMeshBuilder.cpp:596-622).
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/bpsx.h"
#include "dt_format.h"
#include "errors.h"

namespace bpsx {
namespace {

// ---------------------------------------------------------------- RNG (splitmix64)
struct Rng {
  uint64_t s;
  explicit Rng(uint64_t seed) : s(seed * 0x9E3779B97F4A7C15ull + 0x1234567ull) {}
  uint64_t next() {
    uint64_t z = (s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
  }
  // uniform in [0,1)
  double uni() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
  int range(int lo, int hi) {  // inclusive
    if (hi <= lo) return lo;
    return lo + (int)(next() % (uint64_t)(hi - lo + 1));
  }
};

// ---------------------------------------------------------------- BV tree
struct BVItem {
  uint16_t bmin[3], bmax[3];
  int32_t i;
};

void subdivide(std::vector<BVItem>& items, int imin, int imax, int& cur, TileBVNode* nodes) {
  const int inum = imax - imin;
  const int icur = cur;
  TileBVNode& node = nodes[cur++];
  if (inum == 1) {
    for (int a = 0; a < 3; ++a) {
      node.bmin[a] = items[imin].bmin[a];
      node.bmax[a] = items[imin].bmax[a];
    }
    node.i = items[imin].i;
    return;
  }
  for (int a = 0; a < 3; ++a) {
    node.bmin[a] = items[imin].bmin[a];
    node.bmax[a] = items[imin].bmax[a];
  }
  for (int k = imin + 1; k < imax; ++k)
    for (int a = 0; a < 3; ++a) {
      node.bmin[a] = std::min(node.bmin[a], items[k].bmin[a]);
      node.bmax[a] = std::max(node.bmax[a], items[k].bmax[a]);
    }
  const uint16_t ex = node.bmax[0] - node.bmin[0];
  const uint16_t ey = node.bmax[1] - node.bmin[1];
  const uint16_t ez = node.bmax[2] - node.bmin[2];
  int axis = 0;
  uint16_t mx = ex;
  if (ey > mx) { axis = 1; mx = ey; }
  if (ez > mx) axis = 2;
  // glibc's qsort is a merge sort for arrays of this size, i.e. stable.
  std::stable_sort(items.begin() + imin, items.begin() + imax,
                   [axis](const BVItem& a, const BVItem& b) { return a.bmin[axis] < b.bmin[axis]; });
  const int isplit = imin + inum / 2;
  subdivide(items, imin, isplit, cur, nodes);
  subdivide(items, isplit, imax, cur, nodes);
  node.i = -(cur - icur);
}

int pack_tile(const bpsx_tile_desc& d, std::vector<uint8_t>& out) {
  if (!d.verts || !d.polys || !d.poly_flags || !d.poly_areas) return fail(BPSX_E_INVAL, "pack_tile: null input");
  if (d.nvp < 3 || d.nvp > (uint32_t)kMaxVertsPerPoly) return fail(BPSX_E_INVAL, "pack_tile: nvp must be 3..6");
  if (d.vert_count == 0 || d.vert_count >= 0xffff) return fail(BPSX_E_INVAL, "pack_tile: vertex count must be 1..65534");
  if (d.poly_count == 0 || d.poly_count > 0x7fff) return fail(BPSX_E_INVAL, "pack_tile: polygon count must be 1..32767");
  const int nvp = (int)d.nvp;
  const int np = (int)d.poly_count;

  int edgeCount = 0, portalCount = 0, detailTriCount = 0;
  for (int i = 0; i < np; ++i) {
    const uint16_t* p = &d.polys[(size_t)i * 2 * nvp];
    int nv = 0;
    for (int j = 0; j < nvp; ++j) {
      if (p[j] == 0xffff) break;
      if (p[j] >= d.vert_count) return fail(BPSX_E_INVAL, "pack_tile: vertex index out of range");
      nv++;
      edgeCount++;
      const uint16_t nei = p[nvp + j];
      if (nei & 0x8000) {
        if ((nei & 0xf) != 0xf) portalCount++;
      } else if (nei >= d.poly_count) {
        return fail(BPSX_E_INVAL, "pack_tile: neighbour index out of range");
      }
    }
    if (nv < 3) return fail(BPSX_E_INVAL, "pack_tile: polygon with fewer than 3 vertices");
    detailTriCount += nv - 2;
  }
  const int maxLinkCount = edgeCount + portalCount * 2;
  const int bvNodeCount = d.build_bv_tree ? np * 2 : 0;

  const int headerSize = align4(sizeof(TileHeader));
  const int vertsSize = align4(sizeof(float) * 3 * d.vert_count);
  const int polysSize = align4(sizeof(TilePoly) * np);
  const int linksSize = align4(sizeof(TileLink) * maxLinkCount);
  const int dmeshSize = align4(sizeof(TilePolyDetail) * np);
  const int dvertsSize = 0;
  const int dtrisSize = align4(4 * detailTriCount);
  const int bvSize = align4(sizeof(TileBVNode) * bvNodeCount);
  const int total = headerSize + vertsSize + polysSize + linksSize + dmeshSize + dvertsSize + dtrisSize + bvSize;
  out.assign((size_t)total, 0);

  uint8_t* p = out.data();
  TileHeader* h = reinterpret_cast<TileHeader*>(p); p += headerSize;
  float* nverts = reinterpret_cast<float*>(p); p += vertsSize;
  TilePoly* npolys = reinterpret_cast<TilePoly*>(p); p += polysSize;
  p += linksSize;
  TilePolyDetail* ndm = reinterpret_cast<TilePolyDetail*>(p); p += dmeshSize;
  uint8_t* ntris = p; p += dtrisSize;
  TileBVNode* nbv = reinterpret_cast<TileBVNode*>(p);

  h->magic = kTileMagic;
  h->version = kTileVersion;
  h->x = d.tile_x; h->y = d.tile_y; h->layer = d.tile_layer;
  h->userId = 0;
  h->polyCount = np;
  h->vertCount = (int)d.vert_count;
  h->maxLinkCount = maxLinkCount;
  h->detailMeshCount = np;
  h->detailVertCount = 0;
  h->detailTriCount = detailTriCount;
  h->bvNodeCount = bvNodeCount;
  h->offMeshConCount = 0;
  h->offMeshBase = np;
  h->walkableHeight = d.walkable_height;
  h->walkableRadius = d.walkable_radius;
  h->walkableClimb = d.walkable_climb;
  for (int a = 0; a < 3; ++a) { h->bmin[a] = d.bmin[a]; h->bmax[a] = d.bmax[a]; }
  h->bvQuantFactor = 1.0f / d.cs;

  for (uint32_t i = 0; i < d.vert_count; ++i) {
    const uint16_t* iv = &d.verts[(size_t)i * 3];
    nverts[i * 3 + 0] = d.bmin[0] + iv[0] * d.cs;
    nverts[i * 3 + 1] = d.bmin[1] + iv[1] * d.ch;
    nverts[i * 3 + 2] = d.bmin[2] + iv[2] * d.cs;
  }

  int tbase = 0;
  for (int i = 0; i < np; ++i) {
    const uint16_t* src = &d.polys[(size_t)i * 2 * nvp];
    TilePoly& q = npolys[i];
    q.flags = d.poly_flags[i];
    q.areaAndType = d.poly_areas[i] & 0x3f;  // type 0 = ground
    q.vertCount = 0;
    for (int j = 0; j < nvp; ++j) {
      if (src[j] == 0xffff) break;
      q.verts[j] = src[j];
      const uint16_t nei = src[nvp + j];
      if (nei & 0x8000) {
        const uint16_t dir = nei & 0xf;
        if (dir == 0xf) q.neis[j] = 0;
        else if (dir == 0) q.neis[j] = kExtLink | 4;
        else if (dir == 1) q.neis[j] = kExtLink | 2;
        else if (dir == 2) q.neis[j] = kExtLink | 0;
        else if (dir == 3) q.neis[j] = kExtLink | 6;
      } else {
        q.neis[j] = nei + 1;
      }
      q.vertCount++;
    }
    const int nv = q.vertCount;
    ndm[i].vertBase = 0;
    ndm[i].vertCount = 0;
    ndm[i].triBase = (uint32_t)tbase;
    ndm[i].triCount = (uint8_t)(nv - 2);
    for (int j = 2; j < nv; ++j) {
      uint8_t* t = &ntris[tbase * 4];
      t[0] = 0;
      t[1] = (uint8_t)(j - 1);
      t[2] = (uint8_t)j;
      t[3] = (1 << 2);
      if (j == 2) t[3] |= (1 << 0);
      if (j == nv - 1) t[3] |= (1 << 4);
      tbase++;
    }
  }

  if (d.build_bv_tree) {
    std::vector<BVItem> items((size_t)np);
    for (int i = 0; i < np; ++i) {
      const uint16_t* src = &d.polys[(size_t)i * 2 * nvp];
      BVItem& it = items[i];
      it.i = i;
      for (int a = 0; a < 3; ++a) it.bmin[a] = it.bmax[a] = d.verts[(size_t)src[0] * 3 + a];
      for (int j = 1; j < nvp; ++j) {
        if (src[j] == 0xffff) break;
        for (int a = 0; a < 3; ++a) {
          const uint16_t v = d.verts[(size_t)src[j] * 3 + a];
          it.bmin[a] = std::min(it.bmin[a], v);
          it.bmax[a] = std::max(it.bmax[a], v);
        }
      }
      it.bmin[1] = (uint16_t)floorf((float)it.bmin[1] * d.ch / d.cs);
      it.bmax[1] = (uint16_t)ceilf((float)it.bmax[1] * d.ch / d.cs);
    }
    int cur = 0;
    subdivide(items, 0, np, cur, nbv);
  }
  return BPSX_OK;
}

// ---------------------------------------------------------------- floor plans
constexpr float kCs = 0.05f;  // voxel size in metres (north-star configs: cell 0.05 m)
constexpr float kCh = 0.05f;

struct Grid {
  int nx = 0, nz = 0;
  std::vector<uint8_t> w;  // 1 = walkable
  std::vector<uint8_t> keep;  // 1 = never carve (doorways and their approach)
  void init(int x, int z, uint8_t v) {
    nx = x; nz = z;
    w.assign((size_t)x * z, v);
    keep.assign((size_t)x * z, 0);
  }
  bool in(int x, int z) const { return x >= 0 && z >= 0 && x < nx && z < nz; }
  uint8_t& at(int x, int z) { return w[(size_t)z * nx + x]; }
  uint8_t get(int x, int z) const { return in(x, z) ? w[(size_t)z * nx + x] : 0; }
  void fill(int x0, int z0, int x1, int z1, uint8_t v) {  // half-open
    for (int z = std::max(0, z0); z < std::min(nz, z1); ++z)
      for (int x = std::max(0, x0); x < std::min(nx, x1); ++x) at(x, z) = v;
  }
  void protect(int x0, int z0, int x1, int z1) {
    for (int z = std::max(0, z0); z < std::min(nz, z1); ++z)
      for (int x = std::max(0, x0); x < std::min(nx, x1); ++x) keep[(size_t)z * nx + x] = 1;
  }
  int count() const {
    int c = 0;
    for (uint8_t v : w) c += v;
    return c;
  }
  // Keeps only the largest 4-connected walkable component.
  void keep_largest_component() {
    std::vector<int> comp((size_t)nx * nz, -1);
    std::vector<int> stack;
    int best = -1, bestSize = 0, ncomp = 0;
    for (int s = 0; s < nx * nz; ++s) {
      if (!w[s] || comp[s] >= 0) continue;
      int size = 0;
      stack.push_back(s);
      comp[s] = ncomp;
      while (!stack.empty()) {
        const int c = stack.back();
        stack.pop_back();
        size++;
        const int cx = c % nx, cz = c / nx;
        const int dx[4] = {1, -1, 0, 0}, dz[4] = {0, 0, 1, -1};
        for (int k = 0; k < 4; ++k) {
          const int x = cx + dx[k], z = cz + dz[k];
          if (!in(x, z)) continue;
          const int n = z * nx + x;
          if (w[n] && comp[n] < 0) { comp[n] = ncomp; stack.push_back(n); }
        }
      }
      if (size > bestSize) { bestSize = size; best = ncomp; }
      ncomp++;
    }
    for (int s = 0; s < nx * nz; ++s)
      if (w[s] && comp[s] != best) w[s] = 0;
  }
};

int cells_of(float metres, int cell) {
  return std::max(1, (int)lroundf(metres / (kCs * (float)cell)));
}

void carve_boxes(Grid& g, Rng& rng, int cell, float bmin, float bmax, int count, double target_frac) {
  const int floor0 = g.count();
  int carved = 0, placed = 0, guard = 0;
  while (guard++ < 100000) {
    if (count >= 0 && placed >= count) break;
    if (count < 0 && (double)carved >= target_frac * (double)floor0) break;
    const int bx = cells_of((float)(bmin + (bmax - bmin) * rng.uni()), cell);
    const int bz = cells_of((float)(bmin + (bmax - bmin) * rng.uni()), cell);
    const int x0 = rng.range(0, std::max(0, g.nx - bx));
    const int z0 = rng.range(0, std::max(0, g.nz - bz));
    bool ok = true;
    int n = 0;
    for (int z = z0; z < std::min(g.nz, z0 + bz) && ok; ++z)
      for (int x = x0; x < std::min(g.nx, x0 + bx); ++x) {
        if (g.keep[(size_t)z * g.nx + x]) { ok = false; break; }
        n += g.w[(size_t)z * g.nx + x];
      }
    if (!ok || n == 0) continue;
    g.fill(x0, z0, x0 + bx, z0 + bz, 0);
    carved += n;
    placed++;
  }
}

void gen_box_room(const bpsx_scene_params& p, Grid& g, Rng& rng) {
  const int cell = (int)p.cell;
  g.init(cells_of(p.size_x, cell), cells_of(p.size_z, cell), 1);
  carve_boxes(g, rng, cell, p.box_min, p.box_max, (int)p.num_boxes, 0.0);
  g.keep_largest_component();
}

struct DSU {
  std::vector<int> p;
  explicit DSU(int n) : p(n) { for (int i = 0; i < n; ++i) p[i] = i; }
  int find(int a) { while (p[a] != a) a = p[a] = p[p[a]]; return a; }
  bool unite(int a, int b) { a = find(a); b = find(b); if (a == b) return false; p[a] = b; return true; }
};

void gen_rooms(const bpsx_scene_params& p, Grid& g, Rng& rng) {
  const int cell = (int)p.cell;
  const int nrooms = rng.range((int)p.rooms_min, (int)p.rooms_max);
  const int cols = (int)ceil(sqrt((double)nrooms));
  const int rows = (nrooms + cols - 1) / cols;
  const int wt = cells_of(p.wall > 0 ? p.wall : 0.2f, cell);
  const int door = cells_of(p.door_width, cell);
  const int rmin = cells_of(p.room_min, cell), rmax = cells_of(p.room_max, cell);
  std::vector<int> cw(cols), rh(rows), cx(cols), rz(rows);
  int x = wt;
  for (int c = 0; c < cols; ++c) { cw[c] = std::max(door + 2, rng.range(rmin, rmax)); cx[c] = x; x += cw[c] + wt; }
  int z = wt;
  for (int r = 0; r < rows; ++r) { rh[r] = std::max(door + 2, rng.range(rmin, rmax)); rz[r] = z; z += rh[r] + wt; }
  g.init(x, z, 0);
  auto present = [&](int r, int c) { return r >= 0 && c >= 0 && r < rows && c < cols && r * cols + c < nrooms; };
  for (int r = 0; r < rows; ++r)
    for (int c = 0; c < cols; ++c)
      if (present(r, c)) g.fill(cx[c], rz[r], cx[c] + cw[c], rz[r] + rh[r], 1);
  // adjacency list: (room a, room b, horizontal?)
  struct Adj { int r, c, horiz; };
  std::vector<Adj> adj;
  for (int r = 0; r < rows; ++r)
    for (int c = 0; c < cols; ++c) {
      if (!present(r, c)) continue;
      if (present(r, c + 1)) adj.push_back({r, c, 1});
      if (present(r + 1, c)) adj.push_back({r, c, 0});
    }
  for (size_t i = adj.size(); i > 1; --i) std::swap(adj[i - 1], adj[rng.next() % i]);
  DSU dsu(rows * cols);
  for (const Adj& a : adj) {
    const int ia = a.r * cols + a.c;
    const int ib = a.horiz ? ia + 1 : ia + cols;
    const bool tree = dsu.unite(ia, ib);
    if (!tree && rng.uni() >= 0.3) continue;
    if (a.horiz) {
      const int z0 = rz[a.r] + rng.range(0, rh[a.r] - door);
      const int x0 = cx[a.c] + cw[a.c];
      g.fill(x0, z0, x0 + wt, z0 + door, 1);
      g.protect(x0 - 2, z0, x0 + wt + 2, z0 + door);
    } else {
      const int x0 = cx[a.c] + rng.range(0, cw[a.c] - door);
      const int z0 = rz[a.r] + rh[a.r];
      g.fill(x0, z0, x0 + door, z0 + wt, 1);
      g.protect(x0, z0 - 2, x0 + door, z0 + wt + 2);
    }
  }
  if (p.clutter_frac > 0)
    carve_boxes(g, rng, cell, p.box_min > 0 ? p.box_min : 0.5f, p.box_max > 0 ? p.box_max : 1.5f, -1, p.clutter_frac);
  g.keep_largest_component();
}

void gen_maze(const bpsx_scene_params& p, Grid& g, Rng& rng) {
  const int cell = (int)p.cell;
  const int W = std::max(2, (int)p.maze_w), H = std::max(2, (int)p.maze_h);
  const int cmin = cells_of(p.corridor_min, cell), cmax = cells_of(p.corridor_max, cell);
  const int wt = cells_of(p.wall > 0 ? p.wall : 0.5f, cell);
  std::vector<int> wx(W), wz(H), ox(W), oz(H);
  int x = wt;
  for (int i = 0; i < W; ++i) { wx[i] = rng.range(cmin, cmax); ox[i] = x; x += wx[i] + wt; }
  int z = wt;
  for (int k = 0; k < H; ++k) { wz[k] = rng.range(cmin, cmax); oz[k] = z; z += wz[k] + wt; }
  g.init(x, z, 0);
  // spanning tree by randomized depth-first search, then braid
  std::vector<uint8_t> seen((size_t)W * H, 0);
  std::vector<uint8_t> openE((size_t)W * H, 0), openS((size_t)W * H, 0);
  std::vector<int> stack;
  stack.push_back(rng.range(0, W * H - 1));
  seen[stack.back()] = 1;
  while (!stack.empty()) {
    const int c = stack.back();
    const int cxm = c % W, czm = c / W;
    int cand[4], nc = 0;
    if (cxm + 1 < W && !seen[c + 1]) cand[nc++] = 0;
    if (cxm > 0 && !seen[c - 1]) cand[nc++] = 1;
    if (czm + 1 < H && !seen[c + W]) cand[nc++] = 2;
    if (czm > 0 && !seen[c - W]) cand[nc++] = 3;
    if (!nc) { stack.pop_back(); continue; }
    const int d = cand[rng.next() % nc];
    int n;
    if (d == 0) { openE[c] = 1; n = c + 1; }
    else if (d == 1) { openE[c - 1] = 1; n = c - 1; }
    else if (d == 2) { openS[c] = 1; n = c + W; }
    else { openS[c - W] = 1; n = c - W; }
    seen[n] = 1;
    stack.push_back(n);
  }
  for (int c = 0; c < W * H; ++c) {
    if (c % W + 1 < W && !openE[c] && rng.uni() < p.braid) openE[c] = 1;
    if (c / W + 1 < H && !openS[c] && rng.uni() < p.braid) openS[c] = 1;
  }
  for (int k = 0; k < H; ++k)
    for (int i = 0; i < W; ++i) {
      g.fill(ox[i], oz[k], ox[i] + wx[i], oz[k] + wz[k], 1);
      if (openE[k * W + i]) g.fill(ox[i] + wx[i], oz[k], ox[i + 1], oz[k] + wz[k], 1);
      if (openS[k * W + i]) g.fill(ox[i], oz[k] + wz[k], ox[i] + wx[i], oz[k + 1], 1);
    }
}

// Turns the walkable cells into convex polygons (squares, triangle pairs, 2x1 hexagons with
// collinear mid-edge vertices) with shared-edge adjacency and packs them as tiles_x * tiles_z
// tiles; polygon edges on a tile border that face a walkable cell become portals.
int grid_to_mset(const Grid& g, const bpsx_scene_params& p, Rng& rng, std::vector<uint8_t>& mset) {
  const int nx = g.nx, nz = g.nz, cell = (int)p.cell;
  const int ntx = std::max(1, (int)p.tiles_x), ntz = std::max(1, (int)p.tiles_z);
  const int tw = (nx + ntx - 1) / ntx, th = (nz + ntz - 1) / ntz;  // tile size in cells
  if ((long)tw * cell > 65000 || (long)th * cell > 65000) return fail(BPSX_E_INVAL, "gen_scene: tile too large for 16-bit vertices");
  std::vector<std::vector<uint8_t>> tiles;
  uint32_t maxPolys = 0;
  // cell sides: 0 = x- (west), 1 = z+ , 2 = x+ (east), 3 = z-
  std::vector<int32_t> sidePoly((size_t)nx * nz * 4, -1);
  std::vector<uint8_t> used((size_t)nx * nz, 0);
  const int odx[4] = {-1, 0, 1, 0}, odz[4] = {0, 1, 0, -1};
  for (int tz = 0; tz < ntz; ++tz)
    for (int tx = 0; tx < ntx; ++tx) {
      const int x0 = tx * tw, x1 = std::min(nx, x0 + tw), z0 = tz * th, z1 = std::min(nz, z0 + th);
      std::vector<int32_t> vmap((size_t)(tw + 1) * (th + 1), -1);
      std::vector<uint16_t> verts;
      struct P { int nv; int32_t v[6]; int32_t nei[6]; int cx[6], cz[6], side[6]; };
      std::vector<P> polys;
      auto vid = [&](int ix, int iz) {
        int32_t& m = vmap[(size_t)(iz - z0) * (tw + 1) + (ix - x0)];
        if (m < 0) {
          m = (int32_t)(verts.size() / 3);
          verts.push_back((uint16_t)((ix - x0) * cell));
          verts.push_back(0);
          verts.push_back((uint16_t)((iz - z0) * cell));
        }
        return m;
      };
      auto own = [&](int x, int z, int side, int poly) { sidePoly[((size_t)z * nx + x) * 4 + side] = poly; };
      for (int z = z0; z < z1; ++z)
        for (int x = x0; x < x1; ++x) {
          if (!g.get(x, z) || used[(size_t)z * nx + x]) continue;
          used[(size_t)z * nx + x] = 1;
          const double r = rng.uni();
          if (r < p.hex_frac && x + 1 < x1 && g.get(x + 1, z) && !used[(size_t)z * nx + x + 1]) {
            used[(size_t)z * nx + x + 1] = 1;
            // (x1,z0),(x0,z0),(x0,z1),(x1,z1),(x2,z1),(x2,z0): every fan triangle from
            // vertex 0 has positive area.
            P q{}; q.nv = 6;
            const int id = (int)polys.size();
            q.v[0] = vid(x + 1, z);     q.v[1] = vid(x, z);         q.v[2] = vid(x, z + 1);
            q.v[3] = vid(x + 1, z + 1); q.v[4] = vid(x + 2, z + 1); q.v[5] = vid(x + 2, z);
            const int ecx[6] = {x, x, x, x + 1, x + 1, x + 1};
            const int esd[6] = {3, 0, 1, 1, 2, 3};
            for (int e = 0; e < 6; ++e) { q.nei[e] = -1; q.cx[e] = ecx[e]; q.cz[e] = z; q.side[e] = esd[e]; own(ecx[e], z, esd[e], id); }
            polys.push_back(q);
          } else if (r < p.hex_frac + p.tri_frac) {
            const int id = (int)polys.size();
            P a{}, b{}; a.nv = b.nv = 3;
            for (int e = 0; e < 6; ++e) { a.nei[e] = b.nei[e] = -1; a.side[e] = b.side[e] = -1; }
            if (rng.next() & 1) {
              a.v[0] = vid(x, z); a.v[1] = vid(x, z + 1); a.v[2] = vid(x + 1, z + 1);
              a.side[0] = 0; a.side[1] = 1; a.nei[2] = id + 1;
              b.v[0] = vid(x, z); b.v[1] = vid(x + 1, z + 1); b.v[2] = vid(x + 1, z);
              b.nei[0] = id; b.side[1] = 2; b.side[2] = 3;
            } else {
              a.v[0] = vid(x, z); a.v[1] = vid(x, z + 1); a.v[2] = vid(x + 1, z);
              a.side[0] = 0; a.nei[1] = id + 1; a.side[2] = 3;
              b.v[0] = vid(x, z + 1); b.v[1] = vid(x + 1, z + 1); b.v[2] = vid(x + 1, z);
              b.side[0] = 1; b.side[1] = 2; b.nei[2] = id;
            }
            for (int e = 0; e < 3; ++e) {
              a.cx[e] = b.cx[e] = x; a.cz[e] = b.cz[e] = z;
              if (a.side[e] >= 0) own(x, z, a.side[e], id);
              if (b.side[e] >= 0) own(x, z, b.side[e], id + 1);
            }
            polys.push_back(a);
            polys.push_back(b);
          } else {
            P q{}; q.nv = 4;
            const int id = (int)polys.size();
            q.v[0] = vid(x, z); q.v[1] = vid(x, z + 1); q.v[2] = vid(x + 1, z + 1); q.v[3] = vid(x + 1, z);
            for (int e = 0; e < 4; ++e) { q.nei[e] = -1; q.cx[e] = x; q.cz[e] = z; q.side[e] = e; own(x, z, e, id); }
            polys.push_back(q);
          }
        }
      if (polys.empty()) continue;  // a tile without floor is not stored
      if (polys.size() > 0x7fff) return fail(BPSX_E_INVAL, "gen_scene: more than 32767 polygons in a tile; use more tiles or larger cells");
      if (verts.size() / 3 >= 0xffff) return fail(BPSX_E_INVAL, "gen_scene: too many vertices in a tile");
      const int np = (int)polys.size();
      std::vector<uint16_t> pk((size_t)np * 12, 0xffff);
      std::vector<uint16_t> flags((size_t)np, kPolyFlagWalk);
      std::vector<uint8_t> areas((size_t)np, 0);
      for (int i = 0; i < np; ++i) {
        P& q = polys[i];
        for (int e = 0; e < q.nv; ++e) {
          pk[(size_t)i * 12 + e] = (uint16_t)q.v[e];
          uint16_t code = 0xffff;
          if (q.nei[e] >= 0) {
            code = (uint16_t)q.nei[e];
          } else if (q.side[e] >= 0) {
            const int ax = q.cx[e] + odx[q.side[e]], az = q.cz[e] + odz[q.side[e]];
            if (g.in(ax, az) && g.get(ax, az)) {
              if (ax >= x0 && ax < x1 && az >= z0 && az < z1) code = (uint16_t)sidePoly[((size_t)az * nx + ax) * 4 + ((q.side[e] + 2) & 3)];
              else code = (uint16_t)(0x8000 | q.side[e]);  // portal: 0 x-, 1 z+, 2 x+, 3 z-
            }
          }
          pk[(size_t)i * 12 + 6 + e] = code;
        }
      }
      bpsx_tile_desc d{};
      d.verts = verts.data();
      d.vert_count = (uint32_t)(verts.size() / 3);
      d.polys = pk.data();
      d.poly_flags = flags.data();
      d.poly_areas = areas.data();
      d.poly_count = (uint32_t)np;
      d.nvp = 6;
      d.walkable_height = 0.88f;
      d.walkable_radius = 0.18f;
      d.walkable_climb = 0.2f;
      d.cs = kCs; d.ch = kCh;
      d.bmin[0] = p.origin[0] + (float)(x0 * cell) * kCs; d.bmin[1] = p.origin[1]; d.bmin[2] = p.origin[2] + (float)(z0 * cell) * kCs;
      d.bmax[0] = d.bmin[0] + (float)(tw * cell) * kCs;
      d.bmax[1] = p.origin[1] + 1.0f;
      d.bmax[2] = d.bmin[2] + (float)(th * cell) * kCs;
      d.tile_x = tx; d.tile_y = tz; d.tile_layer = 0;
      d.build_bv_tree = 1;
      std::vector<uint8_t> tile;
      const int rc = pack_tile(d, tile);
      if (rc) return rc;
      maxPolys = std::max(maxPolys, (uint32_t)np);
      tiles.push_back(std::move(tile));
    }
  if (tiles.empty()) return fail(BPSX_E_INVAL, "gen_scene: no walkable cells");
  std::vector<const uint8_t*> tp;
  std::vector<size_t> ts;
  for (auto& t : tiles) { tp.push_back(t.data()); ts.push_back(t.size()); }
  uint8_t* o = nullptr; size_t os = 0;
  const float tileW = (float)(tw * cell) * kCs, tileH = (float)(th * cell) * kCs;
  const int rc = bpsx_pack_mset(tp.data(), ts.data(), (uint32_t)tiles.size(), p.origin, tileW, tileH, (uint32_t)tiles.size(),
                                maxPolys, &o, &os);
  if (rc) return rc;
  mset.assign(o, o + os);
  free(o);
  return BPSX_OK;
}

// Parsed view of the first tile(s) of an MSET byte string, enough for host-side sampling.
struct TileView {
  const TileHeader* h;
  const float* verts;
  const TilePoly* polys;
};
int parse_mset(const uint8_t* b, size_t n, std::vector<TileView>& tiles) {
  if (n < sizeof(MsetHeader)) return fail(BPSX_E_INVAL, "navmesh: truncated header");
  MsetHeader mh;
  memcpy(&mh, b, sizeof(mh));
  if (mh.magic != kMsetMagic || mh.version != kMsetVersion) return fail(BPSX_E_INVAL, "navmesh: bad magic/version");
  size_t off = sizeof(MsetHeader);
  for (int t = 0; t < mh.numTiles; ++t) {
    if (off + sizeof(MsetTileHeader) > n) return fail(BPSX_E_INVAL, "navmesh: truncated tile header");
    MsetTileHeader th;
    memcpy(&th, b + off, sizeof(th));
    off += sizeof(th);
    if (!th.tileRef || !th.dataSize) break;
    if (th.dataSize < (int)sizeof(TileHeader) || off + (size_t)th.dataSize > n) return fail(BPSX_E_INVAL, "navmesh: truncated tile");
    const TileHeader* h = reinterpret_cast<const TileHeader*>(b + off);
    if (h->magic != kTileMagic || h->version != kTileVersion) return fail(BPSX_E_INVAL, "navmesh: bad tile magic/version");
    TileView v;
    v.h = h;
    v.verts = reinterpret_cast<const float*>(b + off + align4(sizeof(TileHeader)));
    v.polys = reinterpret_cast<const TilePoly*>(b + off + align4(sizeof(TileHeader)) + align4(12 * h->vertCount));
    tiles.push_back(v);
    off += (size_t)th.dataSize;
  }
  return BPSX_OK;
}

}  // namespace
}  // namespace bpsx

using namespace bpsx;

extern "C" {

int bpsx_pack_tile(const bpsx_tile_desc* desc, uint8_t** out, size_t* out_size) {
  if (!desc || !out || !out_size) return fail(BPSX_E_INVAL, "pack_tile: null argument");
  std::vector<uint8_t> buf;
  const int rc = pack_tile(*desc, buf);
  if (rc) return rc;
  *out = (uint8_t*)malloc(buf.size());
  if (!*out) return fail(BPSX_E_INVAL, "pack_tile: out of memory");
  memcpy(*out, buf.data(), buf.size());
  *out_size = buf.size();
  return BPSX_OK;
}

int bpsx_pack_mset(const uint8_t* const* tiles, const size_t* tile_sizes, uint32_t num_tiles,
                   const float orig[3], float tile_width, float tile_height, uint32_t max_tiles,
                   uint32_t max_polys, uint8_t** out, size_t* out_size) {
  if (!tiles || !tile_sizes || !num_tiles || !orig || !out || !out_size) return fail(BPSX_E_INVAL, "pack_mset: null argument");
  if (num_tiles > max_tiles) return fail(BPSX_E_INVAL, "pack_mset: num_tiles > max_tiles");
  const uint32_t tileBits = ilog2(nextPow2(max_tiles));
  const uint32_t polyBits = ilog2(nextPow2(max_polys));
  if (32 - tileBits - polyBits < 10) return fail(BPSX_E_INVAL, "pack_mset: fewer than 10 salt bits left");
  size_t total = sizeof(MsetHeader);
  for (uint32_t t = 0; t < num_tiles; ++t) total += sizeof(MsetTileHeader) + tile_sizes[t];
  uint8_t* o = (uint8_t*)malloc(total);
  if (!o) return fail(BPSX_E_INVAL, "pack_mset: out of memory");
  MsetHeader mh{};
  mh.magic = kMsetMagic;
  mh.version = kMsetVersion;
  mh.numTiles = (int32_t)num_tiles;
  mh.params.orig[0] = orig[0]; mh.params.orig[1] = orig[1]; mh.params.orig[2] = orig[2];
  mh.params.tileWidth = tile_width;
  mh.params.tileHeight = tile_height;
  mh.params.maxTiles = (int32_t)max_tiles;
  mh.params.maxPolys = (int32_t)max_polys;
  size_t off = 0;
  memcpy(o, &mh, sizeof(mh)); off += sizeof(mh);
  for (uint32_t t = 0; t < num_tiles; ++t) {
    MsetTileHeader th;
    // tile t sits at slot t with salt 1, as a freshly built dtNavMesh would number it
    th.tileRef = (1u << (polyBits + tileBits)) | (t << polyBits);
    th.dataSize = (int32_t)tile_sizes[t];
    memcpy(o + off, &th, sizeof(th)); off += sizeof(th);
    memcpy(o + off, tiles[t], tile_sizes[t]); off += tile_sizes[t];
  }
  *out = o;
  *out_size = total;
  return BPSX_OK;
}

void bpsx_free(void* p) { free(p); }

int bpsx_gen_scene(const bpsx_scene_params* p, uint8_t** out, size_t* out_size) {
  if (!p || !out || !out_size) return fail(BPSX_E_INVAL, "gen_scene: null argument");
  if (p->cell < 1 || p->cell > 40) return fail(BPSX_E_INVAL, "gen_scene: cell must be 1..40 voxels");
  Rng rng(p->seed);
  Grid g;
  switch (p->kind) {
    case BPSX_SCENE_BOX_ROOM: gen_box_room(*p, g, rng); break;
    case BPSX_SCENE_ROOMS: gen_rooms(*p, g, rng); break;
    case BPSX_SCENE_MAZE: gen_maze(*p, g, rng); break;
    default: return fail(BPSX_E_INVAL, "gen_scene: unknown kind");
  }
  std::vector<uint8_t> mset;
  const int rc = grid_to_mset(g, *p, rng, mset);
  if (rc) return rc;
  *out = (uint8_t*)malloc(mset.size());
  if (!*out) return fail(BPSX_E_INVAL, "gen_scene: out of memory");
  memcpy(*out, mset.data(), mset.size());
  *out_size = mset.size();
  return BPSX_OK;
}

int bpsx_sample_points(const void* navmesh_bytes, size_t navmesh_size, uint64_t seed, uint32_t n, float* out_xyz) {
  if (!navmesh_bytes || !out_xyz) return fail(BPSX_E_INVAL, "sample_points: null argument");
  std::vector<TileView> tiles;
  const int rc = parse_mset((const uint8_t*)navmesh_bytes, navmesh_size, tiles);
  if (rc) return rc;
  // cumulative xz area over walkable ground polygons of all tiles
  struct Ref { int tile, poly; };
  std::vector<Ref> refs;
  std::vector<double> cum;
  double acc = 0;
  for (size_t t = 0; t < tiles.size(); ++t)
    for (int i = 0; i < tiles[t].h->polyCount; ++i) {
      const TilePoly& q = tiles[t].polys[i];
      if ((q.areaAndType >> 6) != 0 || !(q.flags & kPolyFlagWalk)) continue;
      const float* v0 = &tiles[t].verts[q.verts[0] * 3];
      double a = 0;
      for (int j = 2; j < q.vertCount; ++j) {
        const float* v1 = &tiles[t].verts[q.verts[j - 1] * 3];
        const float* v2 = &tiles[t].verts[q.verts[j] * 3];
        a += fabs((double)(v2[0] - v0[0]) * (v1[2] - v0[2]) - (double)(v1[0] - v0[0]) * (v2[2] - v0[2])) * 0.5;
      }
      if (a <= 0) continue;
      acc += a;
      refs.push_back({(int)t, i});
      cum.push_back(acc);
    }
  if (refs.empty()) return fail(BPSX_E_INVAL, "sample_points: no walkable polygons");
  Rng rng(seed);
  for (uint32_t k = 0; k < n; ++k) {
    const double r = rng.uni() * acc;
    const size_t idx = std::min(refs.size() - 1, (size_t)(std::upper_bound(cum.begin(), cum.end(), r) - cum.begin()));
    const TileView& tv = tiles[refs[idx].tile];
    const TilePoly& q = tv.polys[refs[idx].poly];
    // pick a fan triangle by area, then a uniform point inside it
    const float* v0 = &tv.verts[q.verts[0] * 3];
    double areas[6], asum = 0;
    for (int j = 2; j < q.vertCount; ++j) {
      const float* v1 = &tv.verts[q.verts[j - 1] * 3];
      const float* v2 = &tv.verts[q.verts[j] * 3];
      areas[j] = fabs((double)(v2[0] - v0[0]) * (v1[2] - v0[2]) - (double)(v1[0] - v0[0]) * (v2[2] - v0[2]));
      asum += areas[j];
    }
    double thr = rng.uni() * asum;
    int tri = q.vertCount - 1;
    for (int j = 2; j < q.vertCount; ++j) {
      if (thr < areas[j]) { tri = j; break; }
      thr -= areas[j];
    }
    const float* v1 = &tv.verts[q.verts[tri - 1] * 3];
    const float* v2 = &tv.verts[q.verts[tri] * 3];
    double a = rng.uni(), b = rng.uni();
    if (a + b > 1) { a = 1 - a; b = 1 - b; }
    // keep a small margin from the triangle boundary so the point is strictly inside
    a = 0.02 + 0.94 * a; b = 0.02 + 0.94 * b;
    if (a + b > 0.98) { const double s = 0.98 / (a + b); a *= s; b *= s; }
    for (int c = 0; c < 3; ++c)
      out_xyz[(size_t)k * 3 + c] = (float)(v0[c] + a * (v1[c] - v0[c]) + b * (v2[c] - v0[c]));
  }
  return BPSX_OK;
}

}  // extern "C"
