// TEST INFRASTRUCTURE — see nav_oracle.h. Compile with -ffp-contract=off: polygon ids must
// match the reference bit for bit, which needs the same fp32 operation order and rounding.
#include "nav_oracle.h"

#include <cfloat>
#include <cmath>
#include <cstring>
#include <limits>
#include <queue>
#include <algorithm>

namespace orc {

void Counters::add(const Counters& o) {
  move_calls += o.move_calls; move_polys += o.move_polys; move_verts += o.move_verts;
  height_tris += o.height_tris; path_calls += o.path_calls; astar_pops += o.astar_pops;
  astar_links += o.astar_links; corridor_polys += o.corridor_polys; snap_calls += o.snap_calls;
  snap_bv_nodes += o.snap_bv_nodes; snap_cands += o.snap_cands;
  snap_cand_verts += o.snap_cand_verts; snap_cand_tris += o.snap_cand_tris;
}

namespace {

// ------------------------------------------------------------------ format constants
constexpr int32_t MSET_MAGIC = ('M' << 24) | ('S' << 16) | ('E' << 8) | 'T';
constexpr int32_t DNAV_MAGIC = ('D' << 24) | ('N' << 16) | ('A' << 8) | 'V';
constexpr int NVP = 6;
constexpr uint16_t EXT_LINK = 0x8000;
constexpr uint32_t NULL_LINK = 0xffffffffu;
constexpr uint16_t FLAG_WALK = 0x01, FLAG_DISABLED = 0x04;
constexpr int TYPE_OFFMESH = 1;

// status bits (DetourStatus.h)
constexpr uint32_t ST_FAILURE = 1u << 31, ST_SUCCESS = 1u << 30, ST_IN_PROGRESS = 1u << 29;
constexpr uint32_t ST_INVALID_PARAM = 1u << 3, ST_BUFFER_TOO_SMALL = 1u << 4, ST_OUT_OF_NODES = 1u << 5,
                   ST_PARTIAL_RESULT = 1u << 6;

struct Poly {
  uint32_t firstLink;
  uint16_t verts[NVP];
  uint16_t neis[NVP];
  uint16_t flags;
  uint8_t vertCount;
  uint8_t areaAndType;
  int type() const { return areaAndType >> 6; }
};
struct Link {
  uint32_t ref, next;
  uint8_t edge, side, bmin, bmax;
};
struct Detail {
  uint32_t vertBase, triBase;
  uint8_t vertCount, triCount;
};
struct BVNode {
  uint16_t bmin[3], bmax[3];
  int32_t i;
};

int align4(int x) { return (x + 3) & ~3; }
uint32_t next_pow2(uint32_t v) {
  v--; v |= v >> 1; v |= v >> 2; v |= v >> 4; v |= v >> 8; v |= v >> 16; v++;
  return v;
}
uint32_t ilog2(uint32_t v) { uint32_t r = 0; while (v >>= 1) r++; return r; }

// ------------------------------------------------------------------ vector helpers
inline void vcopy(float* d, const float* s) { d[0] = s[0]; d[1] = s[1]; d[2] = s[2]; }
inline void vlerp(float* d, const float* a, const float* b, float t) {
  d[0] = a[0] + (b[0] - a[0]) * t;
  d[1] = a[1] + (b[1] - a[1]) * t;
  d[2] = a[2] + (b[2] - a[2]) * t;
}
inline float vdist(const float* a, const float* b) {
  const float dx = b[0] - a[0], dy = b[1] - a[1], dz = b[2] - a[2];
  return sqrtf(dx * dx + dy * dy + dz * dz);
}
inline float vdist_sqr(const float* a, const float* b) {
  const float dx = b[0] - a[0], dy = b[1] - a[1], dz = b[2] - a[2];
  return dx * dx + dy * dy + dz * dz;
}
inline bool vequal(const float* a, const float* b) {
  const float thr = (1.0f / 16384.0f) * (1.0f / 16384.0f);
  return vdist_sqr(a, b) < thr;
}
inline bool vfinite(const float* v) { return std::isfinite(v[0]) && std::isfinite(v[1]) && std::isfinite(v[2]); }
inline bool vfinite2d(const float* v) { return std::isfinite(v[0]) && std::isfinite(v[2]); }
inline float tri_area2d(const float* a, const float* b, const float* c) {
  const float abx = b[0] - a[0], abz = b[2] - a[2];
  const float acx = c[0] - a[0], acz = c[2] - a[2];
  return acx * abz - abx * acz;
}
inline float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }

float dist_pt_seg_sqr2d(const float* pt, const float* p, const float* q, float& t) {
  const float pqx = q[0] - p[0], pqz = q[2] - p[2];
  float dx = pt[0] - p[0], dz = pt[2] - p[2];
  const float d = pqx * pqx + pqz * pqz;
  t = pqx * dx + pqz * dz;
  if (d > 0) t /= d;
  if (t < 0) t = 0;
  else if (t > 1) t = 1;
  dx = p[0] + t * pqx - pt[0];
  dz = p[2] + t * pqz - pt[2];
  return dx * dx + dz * dz;
}

bool point_in_polygon(const float* pt, const float* verts, int nverts) {
  bool c = false;
  for (int i = 0, j = nverts - 1; i < nverts; j = i++) {
    const float* vi = &verts[i * 3];
    const float* vj = &verts[j * 3];
    if (((vi[2] > pt[2]) != (vj[2] > pt[2])) &&
        (pt[0] < (vj[0] - vi[0]) * (pt[2] - vi[2]) / (vj[2] - vi[2]) + vi[0]))
      c = !c;
  }
  return c;
}

bool dist_pt_poly_edges_sqr(const float* pt, const float* verts, int nverts, float* ed, float* et) {
  bool c = false;
  for (int i = 0, j = nverts - 1; i < nverts; j = i++) {
    const float* vi = &verts[i * 3];
    const float* vj = &verts[j * 3];
    if (((vi[2] > pt[2]) != (vj[2] > pt[2])) &&
        (pt[0] < (vj[0] - vi[0]) * (pt[2] - vi[2]) / (vj[2] - vi[2]) + vi[0]))
      c = !c;
    ed[j] = dist_pt_seg_sqr2d(pt, vj, vi, et[j]);
  }
  return c;
}

bool closest_height_point_triangle(const float* p, const float* a, const float* b, const float* c, float& h) {
  const float EPS = 1e-6f;
  float v0[3], v1[3], v2[3];
  for (int k = 0; k < 3; ++k) { v0[k] = c[k] - a[k]; v1[k] = b[k] - a[k]; v2[k] = p[k] - a[k]; }
  float denom = v0[0] * v1[2] - v0[2] * v1[0];
  if (fabsf(denom) < EPS) return false;
  float u = v1[2] * v2[0] - v1[0] * v2[2];
  float v = v0[0] * v2[2] - v0[2] * v2[0];
  if (denom < 0) { denom = -denom; u = -u; v = -v; }
  if (u >= 0.0f && v >= 0.0f && (u + v) <= denom) {
    h = a[1] + (v0[1] * u + v1[1] * v) / denom;
    return true;
  }
  return false;
}

}  // namespace

void random_point_in_convex_poly(const float* pts, int npts, float* areas, float s, float t, float* out) {
  float areasum = 0.0f;
  for (int i = 2; i < npts; i++) {
    areas[i] = tri_area2d(&pts[0], &pts[(i - 1) * 3], &pts[i * 3]);
    areasum += areas[i] > 0.001f ? areas[i] : 0.001f;
  }
  const float thr = s * areasum;
  float acc = 0.0f, u = 1.0f;
  int tri = npts - 1;
  for (int i = 2; i < npts; i++) {
    const float dacc = areas[i];
    if (thr >= acc && thr < (acc + dacc)) {
      u = (thr - acc) / dacc;
      tri = i;
      break;
    }
    acc += dacc;
  }
  const float v = sqrtf(t);
  const float a = 1 - v, b = (1 - u) * v, c = u * v;
  const float* pa = &pts[0];
  const float* pb = &pts[(tri - 1) * 3];
  const float* pc = &pts[tri * 3];
  out[0] = a * pa[0] + b * pb[0] + c * pc[0];
  out[1] = a * pa[1] + b * pb[1] + c * pc[1];
  out[2] = a * pa[2] + b * pb[2] + c * pc[2];
}

// ------------------------------------------------------------------ mesh
class Mesh {
 public:
  // navmesh params
  float orig[3];
  float tileWidth, tileHeight;
  int maxTiles, maxPolys;
  uint32_t tileBits, polyBits, saltBits;
  // the single tile
  uint32_t tileIndex, salt;
  int tx, ty, tlayer;
  int polyCount, vertCount, bvNodeCount;
  float walkableClimb;
  float bmin[3], bmax[3];
  float bvQuantFactor;
  std::vector<float> verts;
  std::vector<Poly> polys;
  std::vector<Link> links;
  std::vector<Detail> details;
  std::vector<float> dverts;
  std::vector<uint8_t> dtris;
  std::vector<BVNode> bv;
  std::vector<int> island;      // per polygon
  std::vector<float> areaCum;   // inclusive float prefix sum of walkable fan areas

  uint32_t refBase() const { return (salt << (polyBits + tileBits)) | (tileIndex << polyBits); }
  // isValidPolyRef (DetourNavMesh.cpp): salt, tile slot and polygon index must all match.
  bool decode(uint32_t ref, int* ip) const {
    if (!ref) return false;
    const uint32_t s = (ref >> (polyBits + tileBits)) & ((1u << saltBits) - 1);
    const uint32_t it = (ref >> polyBits) & ((1u << tileBits) - 1);
    const uint32_t p = ref & ((1u << polyBits) - 1);
    if (it >= (uint32_t)maxTiles || it != tileIndex || s != salt || p >= (uint32_t)polyCount) return false;
    *ip = (int)p;
    return true;
  }
  bool passFilter(const Poly& p) const { return (p.flags & FLAG_WALK) != 0; }  // include WALK, exclude none
  const float* vert(const Poly& p, int k) const { return &verts[(size_t)p.verts[k] * 3]; }
  const float* detailVert(const Poly& p, const Detail& pd, int k) const {
    if (k < p.vertCount) return &verts[(size_t)p.verts[k] * 3];
    return &dverts[(size_t)(pd.vertBase + (k - p.vertCount)) * 3];
  }
};

namespace {

float poly_detail_area(const Mesh& m, int ip) {
  const Poly& p = m.polys[ip];
  const Detail& pd = m.details[ip];
  float area = 0;
  for (int j = 0; j < pd.triCount; ++j) {
    const uint8_t* t = &m.dtris[(size_t)(pd.triBase + j) * 4];
    const float* v[3];
    for (int k = 0; k < 3; ++k) v[k] = m.detailVert(p, pd, t[k]);
    float w1[3], w2[3];
    for (int k = 0; k < 3; ++k) { w1[k] = v[1][k] - v[0][k]; w2[k] = v[2][k] - v[0][k]; }
    const float cx = w1[1] * w2[2] - w1[2] * w2[1];
    const float cy = w1[2] * w2[0] - w1[0] * w2[2];
    const float cz = w1[0] * w2[1] - w1[1] * w2[0];
    const float norm = sqrtf(cx * cx + (cy * cy + cz * cz));
    area = (float)((double)area + 0.5 * (double)norm);
  }
  return area;
}

void build_islands(Mesh& m) {
  m.island.assign((size_t)m.polyCount, -1);
  int next = 0;
  std::vector<int> stack;
  for (int s = 0; s < m.polyCount; ++s) {
    if (m.island[s] >= 0) continue;
    const int id = next++;
    m.island[s] = id;  // the seed is not filter-checked
    stack.push_back(s);
    while (!stack.empty()) {
      const int ip = stack.back();
      stack.pop_back();
      for (uint32_t k = m.polys[ip].firstLink; k != NULL_LINK; k = m.links[k].next) {
        int nb;
        if (!m.decode(m.links[k].ref, &nb)) continue;
        if (m.island[nb] >= 0) continue;
        if (!m.passFilter(m.polys[nb])) continue;
        m.island[nb] = id;
        stack.push_back(nb);
      }
    }
  }
}

}  // namespace

Mesh* mesh_load(const uint8_t* b, size_t n, std::string* err) {
  auto bad = [&](const char* msg) -> Mesh* { if (err) *err = msg; return nullptr; };
  if (n < 40) return bad("truncated MSET header");
  int32_t magic, version, numTiles;
  memcpy(&magic, b, 4); memcpy(&version, b + 4, 4); memcpy(&numTiles, b + 8, 4);
  if (magic != MSET_MAGIC) return bad("bad MSET magic");
  if (version != 1) return bad("bad MSET version");
  Mesh* m = new Mesh();
  memcpy(m->orig, b + 12, 12);
  memcpy(&m->tileWidth, b + 24, 4);
  memcpy(&m->tileHeight, b + 28, 4);
  memcpy(&m->maxTiles, b + 32, 4);
  memcpy(&m->maxPolys, b + 36, 4);
  m->tileBits = ilog2(next_pow2((uint32_t)m->maxTiles));
  m->polyBits = ilog2(next_pow2((uint32_t)m->maxPolys));
  const uint32_t sb = 32 - m->tileBits - m->polyBits;
  m->saltBits = sb < 31 ? sb : 31;
  if (m->saltBits < 10) { delete m; return bad("navmesh params leave fewer than 10 salt bits"); }
  size_t off = 40;
  int loaded = 0;
  for (int t = 0; t < numTiles; ++t) {
    if (off + 8 > n) { delete m; return bad("truncated tile header"); }
    uint32_t tileRef; int32_t dataSize;
    memcpy(&tileRef, b + off, 4); memcpy(&dataSize, b + off + 4, 4);
    off += 8;
    if (!tileRef || !dataSize) break;
    if (dataSize < 100 || off + (size_t)dataSize > n) { delete m; return bad("truncated tile data"); }
    if (loaded) { delete m; return bad("multi-tile navmeshes are not supported by this oracle"); }
    const uint8_t* d = b + off;
    int32_t h[15];
    memcpy(h, d, 60);
    if (h[0] != DNAV_MAGIC) { delete m; return bad("bad tile magic"); }
    if (h[1] != 7) { delete m; return bad("bad tile version"); }
    m->tx = h[2]; m->ty = h[3]; m->tlayer = h[4];
    m->polyCount = h[6]; m->vertCount = h[7];
    const int maxLinkCount = h[8], detailMeshCount = h[9], detailVertCount = h[10], detailTriCount = h[11];
    m->bvNodeCount = h[12];
    const int offMeshConCount = h[13];
    if (offMeshConCount != 0) { delete m; return bad("off-mesh connections are not supported"); }
    memcpy(&m->walkableClimb, d + 68, 4);
    memcpy(m->bmin, d + 72, 12);
    memcpy(m->bmax, d + 84, 12);
    memcpy(&m->bvQuantFactor, d + 96, 4);
    m->tileIndex = (tileRef >> m->polyBits) & ((1u << m->tileBits) - 1);
    m->salt = (tileRef >> (m->polyBits + m->tileBits)) & ((1u << m->saltBits) - 1);
    if (m->tileIndex >= (uint32_t)m->maxTiles) { delete m; return bad("tile index out of range"); }
    const int headerSize = align4(100);
    const int vertsSize = align4(12 * m->vertCount);
    const int polysSize = align4(32 * m->polyCount);
    const int linksSize = align4(12 * maxLinkCount);
    const int dmSize = align4(12 * detailMeshCount);
    const int dvSize = align4(12 * detailVertCount);
    const int dtSize = align4(4 * detailTriCount);
    const int bvSize = align4(16 * m->bvNodeCount);
    if (headerSize + vertsSize + polysSize + linksSize + dmSize + dvSize + dtSize + bvSize > dataSize ||
        detailMeshCount != m->polyCount) { delete m; return bad("tile sections exceed tile size"); }
    const uint8_t* p = d + headerSize;
    m->verts.resize((size_t)m->vertCount * 3);
    memcpy(m->verts.data(), p, (size_t)12 * m->vertCount); p += vertsSize;
    m->polys.resize((size_t)m->polyCount);
    for (int i = 0; i < m->polyCount; ++i) {
      const uint8_t* q = p + (size_t)32 * i;
      Poly& pl = m->polys[i];
      memcpy(&pl.firstLink, q, 4);
      memcpy(pl.verts, q + 4, 12);
      memcpy(pl.neis, q + 16, 12);
      memcpy(&pl.flags, q + 28, 2);
      pl.vertCount = q[30];
      pl.areaAndType = q[31];
      if (pl.vertCount < 3 || pl.vertCount > NVP) { delete m; return bad("polygon vertex count out of range"); }
      for (int k = 0; k < pl.vertCount; ++k)
        if (pl.verts[k] >= m->vertCount) { delete m; return bad("polygon vertex index out of range"); }
    }
    p += polysSize;
    m->links.assign((size_t)maxLinkCount, Link{0, NULL_LINK, 0, 0, 0, 0});
    p += linksSize;
    m->details.resize((size_t)m->polyCount);
    for (int i = 0; i < m->polyCount; ++i) {
      const uint8_t* q = p + (size_t)12 * i;
      memcpy(&m->details[i].vertBase, q, 4);
      memcpy(&m->details[i].triBase, q + 4, 4);
      m->details[i].vertCount = q[8];
      m->details[i].triCount = q[9];
      if ((size_t)m->details[i].triBase + m->details[i].triCount > (size_t)detailTriCount ||
          (size_t)m->details[i].vertBase + m->details[i].vertCount > (size_t)detailVertCount) {
        delete m; return bad("detail mesh out of range");
      }
    }
    p += dmSize;
    m->dverts.resize((size_t)detailVertCount * 3);
    if (detailVertCount) memcpy(m->dverts.data(), p, (size_t)12 * detailVertCount);
    p += dvSize;
    m->dtris.resize((size_t)detailTriCount * 4);
    if (detailTriCount) memcpy(m->dtris.data(), p, (size_t)4 * detailTriCount);
    p += dtSize;
    m->bv.resize((size_t)m->bvNodeCount);
    for (int i = 0; i < m->bvNodeCount; ++i) {
      const uint8_t* q = p + (size_t)16 * i;
      memcpy(m->bv[i].bmin, q, 6);
      memcpy(m->bv[i].bmax, q + 6, 6);
      memcpy(&m->bv[i].i, q + 12, 4);
    }
    off += (size_t)dataSize;
    loaded++;
  }
  if (!loaded) { delete m; return bad("navmesh holds no tile"); }

  // connectIntLinks: the free list hands out link slots 0,1,2,...; edges are linked from
  // the highest index down so each polygon's list runs in ascending edge order.
  uint32_t nextFree = 0;
  const uint32_t base = m->refBase();
  for (int i = 0; i < m->polyCount; ++i) {
    Poly& pl = m->polys[i];
    pl.firstLink = NULL_LINK;
    if (pl.type() == TYPE_OFFMESH) continue;
    for (int j = pl.vertCount - 1; j >= 0; --j) {
      if (pl.neis[j] == 0 || (pl.neis[j] & EXT_LINK)) continue;
      if (nextFree >= m->links.size()) continue;
      Link& l = m->links[nextFree];
      l.ref = base | (uint32_t)(pl.neis[j] - 1);
      l.edge = (uint8_t)j;
      l.side = 0xff;
      l.bmin = l.bmax = 0;
      l.next = pl.firstLink;
      pl.firstLink = nextFree++;
    }
  }
  // removeZeroAreaPolys
  for (int i = 0; i < m->polyCount; ++i)
    if ((double)poly_detail_area(*m, i) < 1e-5) m->polys[i].flags = FLAG_DISABLED;
  build_islands(*m);
  // prefix sums for area-weighted sampling (fan areas as in findRandomPoint)
  m->areaCum.resize((size_t)m->polyCount);
  float acc = 0.0f;
  for (int i = 0; i < m->polyCount; ++i) {
    const Poly& pl = m->polys[i];
    if (pl.type() == 0 && m->passFilter(pl)) {
      float a = 0.0f;
      for (int j = 2; j < pl.vertCount; ++j) a += tri_area2d(m->vert(pl, 0), m->vert(pl, j - 1), m->vert(pl, j));
      if (a > 0.0f) acc += a;
    }
    m->areaCum[i] = acc;
  }
  return m;
}

void mesh_free(Mesh* m) { delete m; }
int mesh_poly_count(const Mesh* m) { return m->polyCount; }
uint32_t mesh_poly_ref(const Mesh* m, int ip) { return m->refBase() | (uint32_t)ip; }
uint16_t mesh_poly_flags(const Mesh* m, int ip) { return m->polys[ip].flags; }
int mesh_poly_island(const Mesh* m, int ip) { return m->island[ip]; }

// ------------------------------------------------------------------ query context
namespace {

constexpr int MAX_NODES = 2048;   // PathFinder.cpp:247
constexpr int HASH_SIZE = 512;    // dtNextPow2(maxNodes/4)
constexpr int MAX_PATH = 256;     // PathFinder.cpp:499
constexpr uint8_t NODE_OPEN = 1, NODE_CLOSED = 2;
constexpr float H_SCALE = 0.999f;

struct Node {
  float pos[3];
  float cost, total;
  uint32_t pidx;  // 1-based index of parent, 0 = none
  uint8_t flags;
  uint32_t id;
};

}  // namespace

struct Query::Impl {
  // A* node pool: lookup by polygon ref, allocation in first-touch order, bounded.
  Node nodes[MAX_NODES];
  uint16_t first[HASH_SIZE];
  uint16_t next[MAX_NODES];
  int nodeCount = 0;
  // open list: binary heap of node indices ordered by total
  uint16_t heap[MAX_NODES + 1];
  int heapSize = 0;

  void clear() { memset(first, 0xff, sizeof(first)); nodeCount = 0; heapSize = 0; }
  static uint32_t hash(uint32_t a) {
    a ^= a >> 16; a *= 0x7feb352du; a ^= a >> 15; a *= 0x846ca68bu; a ^= a >> 16;
    return a;
  }
  Node* getNode(uint32_t id) {
    const uint32_t bucket = hash(id) & (HASH_SIZE - 1);
    for (uint16_t i = first[bucket]; i != 0xffff; i = next[i])
      if (nodes[i].id == id) return &nodes[i];
    if (nodeCount >= MAX_NODES) return nullptr;
    const uint16_t i = (uint16_t)nodeCount++;
    Node& nd = nodes[i];
    nd.pidx = 0; nd.cost = 0; nd.total = 0; nd.id = id; nd.flags = 0;
    next[i] = first[bucket];
    first[bucket] = i;
    return &nd;
  }
  uint32_t idxOf(const Node* nd) const { return nd ? (uint32_t)(nd - nodes) + 1 : 0; }
  Node* at(uint32_t idx) { return idx ? &nodes[idx - 1] : nullptr; }

  void bubbleUp(int i, uint16_t node) {
    int parent = (i - 1) / 2;
    while (i > 0 && nodes[heap[parent]].total > nodes[node].total) {
      heap[i] = heap[parent];
      i = parent;
      parent = (i - 1) / 2;
    }
    heap[i] = node;
  }
  void trickleDown(int i, uint16_t node) {
    int child = i * 2 + 1;
    while (child < heapSize) {
      if (child + 1 < heapSize && nodes[heap[child]].total > nodes[heap[child + 1]].total) child++;
      heap[i] = heap[child];
      i = child;
      child = i * 2 + 1;
    }
    bubbleUp(i, node);
  }
  void push(Node* nd) { heapSize++; bubbleUp(heapSize - 1, (uint16_t)(nd - nodes)); }
  Node* pop() {
    const uint16_t r = heap[0];
    heapSize--;
    trickleDown(0, heap[heapSize]);
    return &nodes[r];
  }
  void modify(Node* nd) {
    const uint16_t id = (uint16_t)(nd - nodes);
    for (int i = 0; i < heapSize; ++i)
      if (heap[i] == id) { bubbleUp(i, id); return; }
  }
};

Query::Query(const Mesh* mesh) : mesh_(mesh), impl_(new Impl()) {}
Query::~Query() { delete impl_; }

namespace {

void collect_verts(const Mesh& m, const Poly& p, float* out) {
  for (int i = 0; i < p.vertCount; ++i) vcopy(&out[i * 3], m.vert(p, i));
}

template <bool onlyBoundary>
void closest_point_on_detail_edges(const Mesh& m, int ip, const float* pos, float* closest) {
  const Poly& p = m.polys[ip];
  const Detail& pd = m.details[ip];
  float dmin = FLT_MAX, tmin = 0;
  const float* pmin = nullptr;
  const float* pmax = nullptr;
  for (int i = 0; i < pd.triCount; i++) {
    const uint8_t* tris = &m.dtris[(size_t)(pd.triBase + i) * 4];
    const int ANY_BOUNDARY = (1 << 0) | (1 << 2) | (1 << 4);
    if (onlyBoundary && (tris[3] & ANY_BOUNDARY) == 0) continue;
    const float* v[3];
    for (int j = 0; j < 3; ++j) v[j] = m.detailVert(p, pd, tris[j]);
    for (int k = 0, j = 2; k < 3; j = k++) {
      const int edgeFlags = (tris[3] >> (j * 2)) & 0x3;
      if ((edgeFlags & 1) == 0 && (onlyBoundary || tris[j] < tris[k])) continue;
      float t;
      const float d = dist_pt_seg_sqr2d(pos, v[j], v[k], t);
      if (d < dmin) { dmin = d; tmin = t; pmin = v[j]; pmax = v[k]; }
    }
  }
  // the reference dereferences pmin/pmax unconditionally; a polygon with no qualifying
  // edge cannot come out of the tile builder, so keep the input position in that case
  if (!pmin) { vcopy(closest, pos); return; }
  vlerp(closest, pmin, pmax, tmin);
}

bool poly_height(const Mesh& m, int ip, const float* pos, float* height, Counters* cnt) {
  const Poly& p = m.polys[ip];
  if (p.type() == TYPE_OFFMESH) return false;
  const Detail& pd = m.details[ip];
  float verts[NVP * 3];
  collect_verts(m, p, verts);
  if (!point_in_polygon(pos, verts, p.vertCount)) return false;
  if (!height) return true;
  if (cnt) cnt->height_tris += pd.triCount;
  for (int j = 0; j < pd.triCount; ++j) {
    const uint8_t* t = &m.dtris[(size_t)(pd.triBase + j) * 4];
    const float* v[3];
    for (int k = 0; k < 3; ++k) v[k] = m.detailVert(p, pd, t[k]);
    float h;
    if (closest_height_point_triangle(pos, v[0], v[1], v[2], h)) { *height = h; return true; }
  }
  float closest[3];
  closest_point_on_detail_edges<false>(m, ip, pos, closest);
  *height = closest[1];
  return true;
}

void closest_point_on_poly(const Mesh& m, int ip, const float* pos, float* closest, bool* over) {
  vcopy(closest, pos);
  if (poly_height(m, ip, pos, &closest[1], nullptr)) { *over = true; return; }
  *over = false;
  closest_point_on_detail_edges<true>(m, ip, pos, closest);
}

void closest_point_on_poly_boundary(const Mesh& m, int ip, const float* pos, float* closest) {
  const Poly& p = m.polys[ip];
  float verts[NVP * 3], edged[NVP], edget[NVP];
  collect_verts(m, p, verts);
  const int nv = p.vertCount;
  if (dist_pt_poly_edges_sqr(pos, verts, nv, edged, edget)) { vcopy(closest, pos); return; }
  float dmin = edged[0];
  int imin = 0;
  for (int i = 1; i < nv; ++i)
    if (edged[i] < dmin) { dmin = edged[i]; imin = i; }
  vlerp(closest, &verts[imin * 3], &verts[((imin + 1) % nv) * 3], edget[imin]);
}

// getPortalPoints for two ground polygons; false when `from` has no link to `to`.
bool portal_points(const Mesh& m, int from, uint32_t toRef, float* left, float* right) {
  const Poly& fp = m.polys[from];
  const Link* link = nullptr;
  for (uint32_t i = fp.firstLink; i != NULL_LINK; i = m.links[i].next)
    if (m.links[i].ref == toRef) { link = &m.links[i]; break; }
  if (!link) return false;
  const float* v0 = m.vert(fp, link->edge);
  const float* v1 = m.vert(fp, (link->edge + 1) % fp.vertCount);
  vcopy(left, v0);
  vcopy(right, v1);
  if (link->side != 0xff && (link->bmin != 0 || link->bmax != 255)) {
    const float s = 1.0f / 255.0f;
    vlerp(left, v0, v1, link->bmin * s);
    vlerp(right, v0, v1, link->bmax * s);
  }
  return true;
}

}  // namespace

// findNearestPoly with half extents {2,4,2} + PathFinder's NaN failure convention.
NavPoint Query::snapPoint(const float* pt) {
  const Mesh& m = *mesh_;
  NavPoint out{{NAN, NAN, NAN}, 0};
  counters.snap_calls++;
  if (!vfinite(pt)) return out;
  const float ext[3] = {2, 4, 2};
  float qmin[3], qmax[3];
  for (int k = 0; k < 3; ++k) { qmin[k] = pt[k] - ext[k]; qmax[k] = pt[k] + ext[k]; }
  const int minx = (int)floorf((qmin[0] - m.orig[0]) / m.tileWidth);
  const int miny = (int)floorf((qmin[2] - m.orig[2]) / m.tileHeight);
  const int maxx = (int)floorf((qmax[0] - m.orig[0]) / m.tileWidth);
  const int maxy = (int)floorf((qmax[2] - m.orig[2]) / m.tileHeight);
  if (m.tx < minx || m.tx > maxx || m.ty < miny || m.ty > maxy) return out;

  float bestD = FLT_MAX;
  uint32_t bestRef = 0;
  float bestPt[3] = {0, 0, 0};
  const uint32_t base = m.refBase();
  auto consider = [&](int ip) {
    const Poly& p = m.polys[ip];
    counters.snap_cands++;
    counters.snap_cand_verts += p.vertCount;
    counters.snap_cand_tris += m.details[ip].triCount;
    float cp[3];
    bool over = false;
    closest_point_on_poly(m, ip, pt, cp, &over);
    const float diff[3] = {pt[0] - cp[0], pt[1] - cp[1], pt[2] - cp[2]};
    float d;
    if (over) {
      d = fabsf(diff[1]) - m.walkableClimb;
      d = d > 0 ? d * d : 0;
    } else {
      d = diff[0] * diff[0] + diff[1] * diff[1] + diff[2] * diff[2];
    }
    if (d < bestD) { vcopy(bestPt, cp); bestD = d; bestRef = base | (uint32_t)ip; }
  };

  if (m.bvNodeCount > 0) {
    const float minx_ = clampf(qmin[0], m.bmin[0], m.bmax[0]) - m.bmin[0];
    const float miny_ = clampf(qmin[1], m.bmin[1], m.bmax[1]) - m.bmin[1];
    const float minz_ = clampf(qmin[2], m.bmin[2], m.bmax[2]) - m.bmin[2];
    const float maxx_ = clampf(qmax[0], m.bmin[0], m.bmax[0]) - m.bmin[0];
    const float maxy_ = clampf(qmax[1], m.bmin[1], m.bmax[1]) - m.bmin[1];
    const float maxz_ = clampf(qmax[2], m.bmin[2], m.bmax[2]) - m.bmin[2];
    const float qf = m.bvQuantFactor;
    uint16_t bmin[3], bmax[3];
    bmin[0] = (uint16_t)(qf * minx_) & 0xfffe;
    bmin[1] = (uint16_t)(qf * miny_) & 0xfffe;
    bmin[2] = (uint16_t)(qf * minz_) & 0xfffe;
    bmax[0] = (uint16_t)(qf * maxx_ + 1) | 1;
    bmax[1] = (uint16_t)(qf * maxy_ + 1) | 1;
    bmax[2] = (uint16_t)(qf * maxz_ + 1) | 1;
    int i = 0;
    while (i < m.bvNodeCount) {
      const BVNode& nd = m.bv[i];
      counters.snap_bv_nodes++;
      bool overlap = true;
      for (int k = 0; k < 3; ++k)
        if (bmin[k] > nd.bmax[k] || bmax[k] < nd.bmin[k]) overlap = false;
      const bool leaf = nd.i >= 0;
      if (leaf && overlap && nd.i < m.polyCount && m.passFilter(m.polys[nd.i])) consider(nd.i);
      if (overlap || leaf) i++;
      else i += -nd.i;
    }
  } else {
    for (int ip = 0; ip < m.polyCount; ++ip) {
      const Poly& p = m.polys[ip];
      if (p.type() == TYPE_OFFMESH || !m.passFilter(p)) continue;
      float bmn[3], bmx[3];
      vcopy(bmn, m.vert(p, 0));
      vcopy(bmx, m.vert(p, 0));
      for (int j = 1; j < p.vertCount; ++j)
        for (int k = 0; k < 3; ++k) {
          const float v = m.vert(p, j)[k];
          if (v < bmn[k]) bmn[k] = v;
          if (v > bmx[k]) bmx[k] = v;
        }
      bool overlap = true;
      for (int k = 0; k < 3; ++k)
        if (qmin[k] > bmx[k] || qmax[k] < bmn[k]) overlap = false;
      if (overlap) consider(ip);
    }
  }
  if (!bestRef) return out;
  vcopy(out.xyz, bestPt);
  // PathFinder tests only x for NaN (projectToPoly, PathFinder.cpp:40)
  if (std::isnan(out.xyz[0])) return NavPoint{{NAN, NAN, NAN}, 0};
  out.ref = bestRef;
  return out;
}

NavPoint Query::tryStep(const NavPoint& start, const float* endPos) {
  const Mesh& m = *mesh_;
  counters.move_calls++;
  int startIp;
  if (!m.decode(start.ref, &startIp) || !vfinite(start.xyz) || !vfinite(endPos)) return start;

  // breadth-first walk bounded by a 64-entry node pool and a 48-entry queue
  constexpr int MAX_STACK = 48, TINY_NODES = 64;
  int nodeId[TINY_NODES];
  bool nodeClosed[TINY_NODES];
  int nnodes = 0;
  int queue[MAX_STACK];
  int nqueue = 0;
  auto getNode = [&](int ip) -> int {
    for (int i = 0; i < nnodes; ++i)
      if (nodeId[i] == ip) return i;
    if (nnodes >= TINY_NODES) return -1;
    nodeId[nnodes] = ip;
    nodeClosed[nnodes] = false;
    return nnodes++;
  };
  const int startNode = getNode(startIp);
  nodeClosed[startNode] = true;
  queue[nqueue++] = startNode;

  float bestPos[3];
  float bestDist = FLT_MAX;
  int bestNode = -1;
  vcopy(bestPos, start.xyz);
  float searchPos[3];
  vlerp(searchPos, start.xyz, endPos, 0.5f);
  const float sr = vdist(start.xyz, endPos) / 2.0f + 0.001f;
  const float searchRadSqr = sr * sr;
  float verts[NVP * 3];

  while (nqueue) {
    const int cur = queue[0];
    for (int i = 0; i < nqueue - 1; ++i) queue[i] = queue[i + 1];
    nqueue--;
    const int curIp = nodeId[cur];
    const Poly& cp = m.polys[curIp];
    const int nverts = cp.vertCount;
    collect_verts(m, cp, verts);
    counters.move_polys++;
    counters.move_verts += nverts;
    if (point_in_polygon(endPos, verts, nverts)) {
      bestNode = cur;
      vcopy(bestPos, endPos);
      break;
    }
    for (int i = 0, j = nverts - 1; i < nverts; j = i++) {
      int neis[8];
      int nneis = 0;
      if (cp.neis[j] & EXT_LINK) {
        for (uint32_t k = cp.firstLink; k != NULL_LINK; k = m.links[k].next) {
          const Link& l = m.links[k];
          int nb;
          if (l.edge == j && l.ref != 0 && m.decode(l.ref, &nb) && m.passFilter(m.polys[nb]) && nneis < 8)
            neis[nneis++] = nb;
        }
      } else if (cp.neis[j]) {
        const int idx = cp.neis[j] - 1;
        if (m.passFilter(m.polys[idx])) neis[nneis++] = idx;
      }
      const float* vj = &verts[j * 3];
      const float* vi = &verts[i * 3];
      if (!nneis) {
        float tseg;
        const float distSqr = dist_pt_seg_sqr2d(endPos, vj, vi, tseg);
        if (distSqr < bestDist) {
          vlerp(bestPos, vj, vi, tseg);
          bestDist = distSqr;
          bestNode = cur;
        }
      } else {
        for (int k = 0; k < nneis; ++k) {
          const int nn = getNode(neis[k]);
          if (nn < 0) continue;
          if (nodeClosed[nn]) continue;
          float tseg;
          const float distSqr = dist_pt_seg_sqr2d(searchPos, vj, vi, tseg);
          if (distSqr > searchRadSqr) continue;
          if (nqueue < MAX_STACK) {
            nodeClosed[nn] = true;
            queue[nqueue++] = nn;
          }
        }
      }
    }
  }
  if (bestNode < 0) return start;  // visitedCount == 0 (PathFinder.cpp:556-558)
  NavPoint out;
  vcopy(out.xyz, bestPos);
  const int lastIp = nodeId[bestNode];
  out.ref = m.refBase() | (uint32_t)lastIp;
  // getPolyHeight(polys[numPolys-1], endPoint, &endPoint[1]); a failure leaves y untouched
  if (vfinite2d(out.xyz)) {
    float h;
    if (poly_height(m, lastIp, out.xyz, &h, &counters)) out.xyz[1] = h;
  }
  return out;
}

float Query::geodesic(const NavPoint& start, const NavPoint& end) {
  const Mesh& m = *mesh_;
  Impl& q = *impl_;
  const float INF = std::numeric_limits<float>::infinity();
  // Eigen isApprox, default precision 1e-5; 3-element sums reduce as a0 + (a1 + a2)
  {
    const float* a = start.xyz;
    const float* b = end.xyz;
    const float d0 = a[0] - b[0], d1 = a[1] - b[1], d2 = a[2] - b[2];
    const float dd = d0 * d0 + (d1 * d1 + d2 * d2);
    const float aa = a[0] * a[0] + (a[1] * a[1] + a[2] * a[2]);
    const float bb = b[0] * b[0] + (b[1] * b[1] + b[2] * b[2]);
    const float prec = 1e-5f;
    const float mn = bb < aa ? bb : aa;  // numext::mini(x, y) = (y < x) ? y : x
    if (dd <= prec * prec * mn) return 0.0f;
  }
  int startIp, endIp;
  if (!m.decode(start.ref, &startIp) || !m.decode(end.ref, &endIp)) return INF;
  if (m.island[startIp] != m.island[endIp]) return INF;

  // ---- findPath
  counters.path_calls++;
  if (!vfinite(start.xyz) || !vfinite(end.xyz)) return INF;
  corridor_.clear();
  uint32_t status;
  if (start.ref == end.ref) {
    corridor_.push_back(start.ref);
    status = ST_SUCCESS;
  } else {
    q.clear();
    Node* startNode = q.getNode(start.ref);
    vcopy(startNode->pos, start.xyz);
    startNode->pidx = 0;
    startNode->cost = 0;
    startNode->total = vdist(start.xyz, end.xyz) * H_SCALE;
    startNode->id = start.ref;
    startNode->flags = NODE_OPEN;
    q.push(startNode);
    Node* lastBest = startNode;
    float lastBestCost = startNode->total;
    bool outOfNodes = false;
    // ---- check of the multi-node pass rules (see Query::PassCheck); no effect on the search
    struct PlanUpd { uint32_t ref; float total; float pos[3]; };
    struct Plan {
      int count = 0, done = 0, first = 0;
      bool pair = false, blind = false;
      int node[8];
      std::vector<PlanUpd> upd[8];
    } plan;
    auto lookup = [&](uint32_t ref) -> Node* {
      const uint32_t bucket = Impl::hash(ref) & (HASH_SIZE - 1);
      for (uint16_t i = q.first[bucket]; i != 0xffff; i = q.next[i])
        if (q.nodes[i].id == ref) return &q.nodes[i];
      return nullptr;
    };
    // what expanding node `best` writes, computed without changing anything: (polygon, total) in link order
    auto dry_run = [&](const Node* best, std::vector<uint32_t>& reads, std::vector<PlanUpd>& upds) {
      const int bestIp = (int)(best->id & ((1u << m.polyBits) - 1));
      uint32_t parentRef = 0;
      if (best->pidx) parentRef = q.at(best->pidx)->id;
      reads.push_back(best->id);
      for (uint32_t li = m.polys[bestIp].firstLink; li != NULL_LINK; li = m.links[li].next) {
        const uint32_t nref = m.links[li].ref;
        if (!nref || nref == parentRef) continue;
        if (!m.passFilter(m.polys[(int)(nref & ((1u << m.polyBits) - 1))])) continue;
        reads.push_back(nref);
        const Node* nn = lookup(nref);
        float npos[3];
        uint8_t flags = 0;
        float ntotal = 0;
        // a polygon may hold two links to one neighbour: the second sees what the first wrote
        const PlanUpd* mine = nullptr;
        for (const PlanUpd& u : upds) if (u.ref == nref) mine = &u;
        if (nn && nn->flags) { vcopy(npos, nn->pos); flags = nn->flags; ntotal = nn->total; }
        if (mine) { vcopy(npos, mine->pos); flags = 1; ntotal = mine->total; }
        if (!flags) {
          float left[3], right[3];
          if (!portal_points(m, bestIp, nref, left, right)) continue;
          for (int k = 0; k < 3; ++k) npos[k] = (left[k] + right[k]) * 0.5f;
        }
        float cost, heuristic;
        if (nref == end.ref) { cost = best->cost + vdist(best->pos, npos) * 1.0f + vdist(npos, end.xyz) * 1.0f; heuristic = 0; }
        else { cost = best->cost + vdist(best->pos, npos) * 1.0f; heuristic = vdist(npos, end.xyz) * H_SCALE; }
        const float total = cost + heuristic;
        if (flags && total >= ntotal) continue;
        upds.push_back({nref, total, {npos[0], npos[1], npos[2]}});
      }
    };
    auto make_plan = [&]() {
      plan = Plan();
      const int rows = (passCheck.rows & 0xff) < 8 ? (passCheck.rows & 0xff) : 8;
      const bool keyRule = !(passCheck.rows & 0x100), readRule = !(passCheck.rows & 0x200);   // switches for the tests that drop a rule
      // the open list sorted by total: the first rows + 1 entries
      std::vector<int> order(q.heapSize);
      for (int i = 0; i < q.heapSize; ++i) order[i] = q.heap[i];
      const int want = q.heapSize < rows + 1 ? q.heapSize : rows + 1;
      std::partial_sort(order.begin(), order.begin() + want, order.end(),
                        [&](int a, int b) { return q.nodes[a].total < q.nodes[b].total; });
      const float INF_KEY = std::numeric_limits<float>::infinity();
      auto key = [&](int j) { return j < q.heapSize ? q.nodes[order[j]].total : INF_KEY; };
      auto below_next = [&](int j) { return j < q.heapSize && (j + 1 >= q.heapSize || key(j) < key(j + 1)); };
      int lim = 0;
      while (lim < rows && below_next(lim)) lim++;
      if (lim == 0) {
        // the first two entries share the smallest total: a pair when the third does not
        if (rows >= 2 && q.heapSize >= 2 && below_next(1)) {
          plan.pair = true;
          lim = 2;
          while (lim < rows && below_next(lim)) lim++;
        } else { plan.blind = true; plan.count = 1; passCheck.ties++; return; }
      }
      for (int j = 0; j < lim; ++j)
        if (q.nodes[order[j]].id == end.ref) { lim = j == 0 ? 1 : j; break; }
      if (plan.pair && lim < 2) { plan = Plan(); plan.blind = true; plan.count = 1; passCheck.ties++; return; }
      std::vector<uint32_t> reads[8];
      for (int j = 0; j < lim; ++j) {
        plan.node[j] = order[j];
        if (q.nodes[order[j]].id != end.ref) dry_run(&q.nodes[order[j]], reads[j], plan.upd[j]);
      }
      // a row depends on an earlier update only through its own node and through the polygons
      // that it updates itself: what it reads and leaves alone only gets a lower total
      for (int j = 0; j < lim; ++j) {
        reads[j].assign(1, q.nodes[order[j]].id);
        for (const PlanUpd& u : plan.upd[j]) reads[j].push_back(u.ref);
      }
      int c = lim;
      for (int j = 1; j < c; ++j) {
        bool stands = true;
        for (int i = 0; i < j && stands; ++i)
          for (const PlanUpd& u : plan.upd[i]) {
            if (keyRule && u.total <= key(j)) { stands = false; break; }
            if (readRule) for (uint32_t r : reads[j]) if (r == u.ref) { stands = false; break; }
            if (!stands) break;
          }
        if (!stands) { c = j; break; }
      }
      if (plan.pair) {
        bool ok = c >= 2;
        for (const PlanUpd& u : plan.upd[1]) {
          if (u.total <= key(1)) ok = false;
          for (uint32_t r : reads[0]) if (r == u.ref) ok = false;
        }
        if (!ok) { plan = Plan(); plan.blind = true; plan.count = 1; passCheck.ties++; return; }
        passCheck.pairs++;
      }
      plan.count = c;
      passCheck.passes++;
      passCheck.nodes += (uint64_t)c;
    };
    std::vector<PlanUpd> actual;
    int checking = -1;   // row of the plan whose expansion is under way
    while (q.heapSize > 0) {
      if (passCheck.rows > 0 && !outOfNodes) {
        if (plan.done == plan.count) make_plan();
        checking = -1;
        if (!plan.blind) {
          const int top = q.heap[0];
          int row = plan.done;
          if (plan.pair && plan.done == 0) row = top == plan.node[1] ? 1 : 0;   // either of the two may come first
          if (plan.pair && plan.done == 1) row = 1 - plan.first;
          if (plan.done == 0) plan.first = row;
          if (top != plan.node[row]) passCheck.wrongNode++;
          checking = row;
          actual.clear();
        }
        plan.done++;
      }
      Node* best = q.pop();
      best->flags &= ~NODE_OPEN;
      best->flags |= NODE_CLOSED;
      if (best->id == end.ref) { lastBest = best; break; }
      counters.astar_pops++;
      const int bestIp = (int)(best->id & ((1u << m.polyBits) - 1));
      const Poly& bp = m.polys[bestIp];
      uint32_t parentRef = 0;
      if (best->pidx) parentRef = q.at(best->pidx)->id;
      for (uint32_t li = bp.firstLink; li != NULL_LINK; li = m.links[li].next) {
        counters.astar_links++;
        const uint32_t nref = m.links[li].ref;
        if (!nref || nref == parentRef) continue;
        const int nIp = (int)(nref & ((1u << m.polyBits) - 1));
        if (!m.passFilter(m.polys[nIp])) continue;
        Node* nn = q.getNode(nref);  // single tile: crossSide is always 0
        if (!nn) { outOfNodes = true; continue; }
        if (nn->flags == 0) {
          float left[3], right[3];
          if (portal_points(m, bestIp, nref, left, right)) {
            nn->pos[0] = (left[0] + right[0]) * 0.5f;
            nn->pos[1] = (left[1] + right[1]) * 0.5f;
            nn->pos[2] = (left[2] + right[2]) * 0.5f;
          }
        }
        float cost, heuristic;
        if (nref == end.ref) {
          const float curCost = vdist(best->pos, nn->pos) * 1.0f;
          const float endCost = vdist(nn->pos, end.xyz) * 1.0f;
          cost = best->cost + curCost + endCost;
          heuristic = 0;
        } else {
          const float curCost = vdist(best->pos, nn->pos) * 1.0f;
          cost = best->cost + curCost;
          heuristic = vdist(nn->pos, end.xyz) * H_SCALE;
        }
        const float total = cost + heuristic;
        if ((nn->flags & NODE_OPEN) && total >= nn->total) continue;
        if ((nn->flags & NODE_CLOSED) && total >= nn->total) continue;
        nn->pidx = q.idxOf(best);
        nn->id = nref;
        nn->flags = (uint8_t)(nn->flags & ~NODE_CLOSED);
        nn->cost = cost;
        nn->total = total;
        if (checking >= 0) actual.push_back({nref, total, {0, 0, 0}});
        if (nn->flags & NODE_OPEN) {
          q.modify(nn);
        } else {
          nn->flags |= NODE_OPEN;
          q.push(nn);
        }
        if (heuristic < lastBestCost) { lastBestCost = heuristic; lastBest = nn; }
      }
      if (checking >= 0 && !outOfNodes) {
        // the expansion wrote what the prediction, made from the state before the pass, said
        const std::vector<PlanUpd>& want = plan.upd[checking];
        bool same = want.size() == actual.size();
        for (size_t i = 0; same && i < want.size(); ++i)
          same = want[i].ref == actual[i].ref && memcmp(&want[i].total, &actual[i].total, 4) == 0;
        if (!same) passCheck.wrongUpdate++;
      }
    }
    // getPathToNode
    int length = 0;
    for (Node* c = lastBest; c; c = q.at(c->pidx)) length++;
    Node* cur = lastBest;
    int writeCount = length;
    for (; writeCount > MAX_PATH; writeCount--) cur = q.at(cur->pidx);
    corridor_.assign((size_t)writeCount, 0);
    for (int i = writeCount - 1; i >= 0; i--) { corridor_[i] = cur->id; cur = q.at(cur->pidx); }
    status = ST_SUCCESS;
    if (length > MAX_PATH) status |= ST_BUFFER_TOO_SMALL;
    if (lastBest->id != end.ref) status |= ST_PARTIAL_RESULT;
    if (outOfNodes) status |= ST_OUT_OF_NODES;
  }
  if (status != ST_SUCCESS || corridor_.empty()) return INF;
  return corridorLength(start, end);
}

// findStraightPath over corridor_ and the summed length of its points (PathFinder.cpp:473-482,
// 512-525; DetourNavMeshQuery.cpp:1765-1994).
float Query::corridorLength(const NavPoint& start, const NavPoint& end) {
  const Mesh& m = *mesh_;
  const float INF = std::numeric_limits<float>::infinity();
  // ---- findStraightPath (options 0, at most 256 points)
  const int pathSize = (int)corridor_.size();
  counters.corridor_polys += (uint64_t)pathSize;
  const uint32_t* path = corridor_.data();
  const uint32_t polyMask = (1u << m.polyBits) - 1;
  float pts[MAX_PATH * 3];
  int npts = 0;
  // appendVertex: returns IN_PROGRESS, SUCCESS or SUCCESS|BUFFER_TOO_SMALL
  auto append = [&](const float* pos, bool isEnd) -> uint32_t {
    if (npts > 0 && vequal(&pts[(npts - 1) * 3], pos)) return ST_IN_PROGRESS;
    vcopy(&pts[npts * 3], pos);
    npts++;
    if (npts >= MAX_PATH) return ST_SUCCESS | ST_BUFFER_TOO_SMALL;
    if (isEnd) return ST_SUCCESS;
    return ST_IN_PROGRESS;
  };
  auto run_funnel = [&]() -> uint32_t {
    float closestStart[3], closestEnd[3];
    int ip0, ipN;
    if (!m.decode(path[0], &ip0)) return ST_FAILURE | ST_INVALID_PARAM;
    closest_point_on_poly_boundary(m, ip0, start.xyz, closestStart);
    if (!m.decode(path[pathSize - 1], &ipN)) return ST_FAILURE | ST_INVALID_PARAM;
    closest_point_on_poly_boundary(m, ipN, end.xyz, closestEnd);
    uint32_t stat = append(closestStart, false);
    if (stat != ST_IN_PROGRESS) return stat;
    if (pathSize > 1) {
      float apex[3], pl[3], pr[3];
      vcopy(apex, closestStart); vcopy(pl, apex); vcopy(pr, apex);
      int apexIndex = 0, leftIndex = 0, rightIndex = 0;
      uint32_t leftRef = path[0], rightRef = path[0];
      for (int i = 0; i < pathSize; ++i) {
        float left[3], right[3];
        if (i + 1 < pathSize) {
          if (!portal_points(m, (int)(path[i] & polyMask), path[i + 1], left, right)) {
            closest_point_on_poly_boundary(m, (int)(path[i] & polyMask), end.xyz, closestEnd);
            append(closestEnd, false);
            return ST_SUCCESS | ST_PARTIAL_RESULT | (npts >= MAX_PATH ? ST_BUFFER_TOO_SMALL : 0);
          }
          if (i == 0) {
            float t;
            if (dist_pt_seg_sqr2d(apex, left, right, t) < 0.001f * 0.001f) continue;
          }
        } else {
          vcopy(left, closestEnd);
          vcopy(right, closestEnd);
        }
        if (tri_area2d(apex, pr, right) <= 0.0f) {
          if (vequal(apex, pr) || tri_area2d(apex, pl, right) > 0.0f) {
            vcopy(pr, right);
            rightRef = (i + 1 < pathSize) ? path[i + 1] : 0;
            rightIndex = i;
          } else {
            vcopy(apex, pl);
            apexIndex = leftIndex;
            stat = append(apex, leftRef == 0);
            if (stat != ST_IN_PROGRESS) return stat;
            vcopy(pl, apex); vcopy(pr, apex);
            leftIndex = apexIndex; rightIndex = apexIndex;
            i = apexIndex;
            continue;
          }
        }
        if (tri_area2d(apex, pl, left) >= 0.0f) {
          if (vequal(apex, pl) || tri_area2d(apex, pr, left) < 0.0f) {
            vcopy(pl, left);
            leftRef = (i + 1 < pathSize) ? path[i + 1] : 0;
            leftIndex = i;
          } else {
            vcopy(apex, pr);
            apexIndex = rightIndex;
            stat = append(apex, rightRef == 0);
            if (stat != ST_IN_PROGRESS) return stat;
            vcopy(pl, apex); vcopy(pr, apex);
            leftIndex = apexIndex; rightIndex = apexIndex;
            i = apexIndex;
            continue;
          }
        }
      }
    }
    append(closestEnd, true);
    return ST_SUCCESS | (npts >= MAX_PATH ? ST_BUFFER_TOO_SMALL : 0);
  };
  const uint32_t fstat = run_funnel();
  if (fstat != ST_SUCCESS || npts == 0) return INF;
  // pathLength: the first term is |p0 - p0| = 0; 3-element norm reduces as x + (y + z)
  float length = 0;
  const float* prev = &pts[0];
  for (int i = 0; i < npts; ++i) {
    const float* p = &pts[i * 3];
    const float dx = prev[0] - p[0], dy = prev[1] - p[1], dz = prev[2] - p[2];
    length += sqrtf(dx * dx + (dy * dy + dz * dz));
    prev = p;
  }
  return length;
}

// NOT a restatement of the reference: the goal-rooted distance-field formulation, for measuring
// how far its distances are from findPath's.  A Dijkstra search from `start` (the goal point)
// over the same graph A* searches (node = polygon, node position = midpoint of the portal
// through which the polygon was first reached, edge cost = distance between node positions)
// gives every polygon a parent towards the goal; the corridor of a query is the parent chain
// from the end point's polygon, and the same string pulling gives the length.  The field is
// kept while consecutive calls have the same start point.
float Query::geodesicViaField(const NavPoint& start, const NavPoint& end) {
  const Mesh& m = *mesh_;
  const float INF = std::numeric_limits<float>::infinity();
  {
    const float* a = start.xyz;
    const float* b = end.xyz;
    const float d0 = a[0] - b[0], d1 = a[1] - b[1], d2 = a[2] - b[2];
    const float dd = d0 * d0 + (d1 * d1 + d2 * d2);
    const float aa = a[0] * a[0] + (a[1] * a[1] + a[2] * a[2]);
    const float bb = b[0] * b[0] + (b[1] * b[1] + b[2] * b[2]);
    const float mn = bb < aa ? bb : aa;
    if (dd <= 1e-5f * 1e-5f * mn) return 0.0f;
  }
  int startIp, endIp;
  if (!m.decode(start.ref, &startIp) || !m.decode(end.ref, &endIp)) return INF;
  if (m.island[startIp] != m.island[endIp]) return INF;
  if (!vfinite(start.xyz) || !vfinite(end.xyz)) return INF;
  const int np = (int)m.polys.size();
  if (field_.parent.size() != (size_t)np || field_.rootRef != start.ref || memcmp(field_.root, start.xyz, 12) != 0) {
    field_.parent.assign((size_t)np, -2);   // -2 not reached, -1 root
    field_.pos.assign((size_t)np * 3, 0.f);
    field_.cost.assign((size_t)np, INF);
    std::vector<uint8_t> closed((size_t)np, 0);
    field_.rootRef = start.ref;
    memcpy(field_.root, start.xyz, 12);
    typedef std::pair<float, int> Item;
    std::priority_queue<Item, std::vector<Item>, std::greater<Item>> open;
    field_.parent[startIp] = -1;
    field_.cost[startIp] = 0;
    vcopy(&field_.pos[(size_t)startIp * 3], start.xyz);
    open.push(Item(0.f, startIp));
    while (!open.empty()) {
      const Item it = open.top();
      open.pop();
      const int bi = it.second;
      if (closed[bi] || it.first != field_.cost[bi]) continue;
      closed[bi] = 1;
      const Poly& bp = m.polys[bi];
      for (uint32_t li = bp.firstLink; li != NULL_LINK; li = m.links[li].next) {
        const uint32_t nref = m.links[li].ref;
        if (!nref) continue;
        const int ni = (int)(nref & ((1u << m.polyBits) - 1));
        if (ni == field_.parent[bi] || !m.passFilter(m.polys[ni]) || closed[ni]) continue;
        float* npos = &field_.pos[(size_t)ni * 3];
        if (field_.parent[ni] == -2) {
          float left[3], right[3];
          if (portal_points(m, bi, nref, left, right)) {
            npos[0] = (left[0] + right[0]) * 0.5f;
            npos[1] = (left[1] + right[1]) * 0.5f;
            npos[2] = (left[2] + right[2]) * 0.5f;
          }
        }
        const float c = field_.cost[bi] + vdist(&field_.pos[(size_t)bi * 3], npos);
        if (c < field_.cost[ni]) {
          field_.cost[ni] = c;
          field_.parent[ni] = bi;
          open.push(Item(c, ni));
        }
      }
    }
  }
  if (field_.parent[endIp] == -2) return INF;
  corridor_.clear();
  for (int c = endIp; c >= 0; c = field_.parent[c]) {
    corridor_.push_back(m.refBase() | (uint32_t)c);
    if ((int)corridor_.size() > MAX_PATH) return INF;   // the reference's corridor buffer holds 256 polygons
  }
  std::reverse(corridor_.begin(), corridor_.end());
  return corridorLength(start, end);
}

bool Query::samplePoint(float u0, float s, float t, float* out_xyz, uint32_t* out_ref) {
  const Mesh& m = *mesh_;
  const int n = m.polyCount;
  const float total = n ? m.areaCum[n - 1] : 0.0f;
  if (!(total > 0.0f)) return false;
  const float target = u0 * total;
  int lo = 0, hi = n - 1;  // first index with areaCum > target, clamped to the last polygon
  while (lo < hi) {
    const int mid = (lo + hi) / 2;
    if (m.areaCum[mid] > target) hi = mid;
    else lo = mid + 1;
  }
  const Poly& p = m.polys[lo];
  float verts[NVP * 3], areas[NVP];
  collect_verts(m, p, verts);
  float pt[3];
  random_point_in_convex_poly(verts, p.vertCount, areas, s, t, pt);
  float h;
  if (vfinite2d(pt) && poly_height(m, lo, pt, &h, nullptr)) pt[1] = h;
  vcopy(out_xyz, pt);
  *out_ref = m.refBase() | (uint32_t)lo;
  return true;
}

}  // namespace orc
