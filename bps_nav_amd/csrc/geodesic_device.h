// Geodesic distance on the GPU: Detour's A* over the polygon graph followed by the funnel
// (string pulling) and the summed segment length, with the exact buffer limits and failure
// conventions of the reference, so that the value equals PathFinder::findPath's.
//
// Execution model: one wavefront (64 lanes) owns one query at a time and pulls the next from
// a shared queue when done.  The whole working set of A* lives in LDS: the open list (a binary
// heap whose pops and pushes are done by all lanes at once, see HeapOps), the hash heads and
// chains of the node pool, and the first kNodesLds nodes; only nodes beyond that and heap
// entries beyond kHeapLds spill to a per-wavefront scratch slot in HBM.  Per expanded node the
// only HBM traffic is the polygon's 128-byte record.  Lane j of the wavefront handles edge j of
// the expanded polygon (node lookup, portal midpoint, cost); heap updates are then applied in
// edge order, which is what makes the result identical to the sequential algorithm, ties
// included.
//
// Reference semantics followed: DetourNavMeshQuery.cpp:945-1178 (findPath, getPathToNode),
// :1661-1696, 1765-1994 (appendVertex, findStraightPath), :2279-2349 (getPortalPoints);
// DetourNode.cpp:50-200 (node pool, heap order); PathFinder.cpp:473-541.
#pragma once
#include "nav_device.h"

namespace bpsx {

#ifdef BPSX_PHASE_TIMING
#define PHASE_MARK(k) do { const unsigned long long now_ = __builtin_readcyclecounter(); phase_acc[k] += now_ - phase_t0; phase_t0 = now_; } while (0)
#else
#define PHASE_MARK(k) do { } while (0)
#endif

constexpr int kNodesLds = 512;   // nodes kept in LDS per query
constexpr int kHeapLds = 384;    // open-list entries kept in LDS per query
constexpr int kHashSize = 512;

BPSX_DEV void wave_sync() {
  // All lanes belong to one wavefront: LDS and memory operations issue in program order, so
  // only the compiler has to be kept from reordering across this point.
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}
BPSX_DEV int uniform_i(int v) { return __builtin_amdgcn_readfirstlane(v); }
BPSX_DEV float lane_f(float v, int lane) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane)); }
BPSX_DEV int lane_i(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }

// LDS of one wavefront.
struct GeoLds {
  float n_total[kNodesLds];
  float n_cost[kNodesLds];
  float n_pos[3][kNodesLds];
  uint32_t n_meta[kNodesLds];      // id:15 | flags:2 << 15 | pidx:12 << 17
  uint16_t n_next[kNodesLds];
  uint16_t first[kHashSize];
  HeapEntry heap[kHeapLds];
};
// After A* the node arrays are dead; the funnel reuses them for the corridor and its portals.
struct FunnelLds {
  float portals[kMaxPath][6];
  uint16_t corridor[kMaxPath];
};
static_assert(sizeof(FunnelLds) <= offsetof(GeoLds, n_meta), "funnel scratch must stay clear of the node links");

BPSX_DEV uint32_t meta_pack(uint32_t id, uint32_t flags, uint32_t pidx) { return id | (flags << 15) | (pidx << 17); }
BPSX_DEV uint32_t meta_id(uint32_t m) { return m & 0x7fffu; }
BPSX_DEV uint32_t meta_flags(uint32_t m) { return (m >> 15) & 3u; }
BPSX_DEV uint32_t meta_pidx(uint32_t m) { return m >> 17; }

struct NodeVal {
  float pos[3];
  float cost, total;
  uint32_t meta;
};

struct GeoWave {
  GeoLds* L;
  GeoSlot* ws;
  int lane;
  int heapSize;
  int nodeCount;

  // ---------------------------------------------------------------- node pool
  BPSX_DEV uint32_t node_meta(int i) const {
    if (i < kNodesLds) return L->n_meta[i];
    const ANode& n = ws->nodes[i];
    return meta_pack(n.id, n.flags, n.pidx);
  }
  BPSX_DEV NodeVal node_load(int i) const {
    NodeVal v;
    if (i < kNodesLds) {
      v.pos[0] = L->n_pos[0][i]; v.pos[1] = L->n_pos[1][i]; v.pos[2] = L->n_pos[2][i];
      v.cost = L->n_cost[i]; v.total = L->n_total[i]; v.meta = L->n_meta[i];
    } else {
      const ANode n = ws->nodes[i];
      v.pos[0] = n.pos[0]; v.pos[1] = n.pos[1]; v.pos[2] = n.pos[2];
      v.cost = n.cost; v.total = n.total; v.meta = meta_pack(n.id, n.flags, n.pidx);
    }
    return v;
  }
  BPSX_DEV void node_store(int i, const NodeVal& v) const {
    if (i < kNodesLds) {
      L->n_pos[0][i] = v.pos[0]; L->n_pos[1][i] = v.pos[1]; L->n_pos[2][i] = v.pos[2];
      L->n_cost[i] = v.cost; L->n_total[i] = v.total; L->n_meta[i] = v.meta;
    } else {
      ANode n;
      n.pos[0] = v.pos[0]; n.pos[1] = v.pos[1]; n.pos[2] = v.pos[2];
      n.cost = v.cost; n.total = v.total;
      n.id = meta_id(v.meta); n.flags = meta_flags(v.meta); n.pidx = meta_pidx(v.meta);
      ws->nodes[i] = n;
    }
  }
  BPSX_DEV void node_set_meta(int i, uint32_t m) const {
    if (i < kNodesLds) L->n_meta[i] = m;
    else { ws->nodes[i].flags = meta_flags(m); ws->nodes[i].pidx = meta_pidx(m); ws->nodes[i].id = meta_id(m); }
  }
  BPSX_DEV int node_next(int i) const { return i < kNodesLds ? L->n_next[i] : ws->next[i]; }
  static BPSX_DEV uint32_t hash(uint32_t a) {
    a ^= a >> 16; a *= 0x7feb352du; a ^= a >> 15; a *= 0x846ca68bu; a ^= a >> 16;
    return a & (kHashSize - 1);
  }
  BPSX_DEV void clear() {
    for (int i = lane; i < kHashSize; i += 64) L->first[i] = 0xffff;
    heapSize = 0;
    nodeCount = 0;
    wave_sync();
  }
  // node index of polygon ip, or -1 (any lane, independently)
  BPSX_DEV int find(uint32_t ip) const {
    for (int i = L->first[hash(ip)]; i != 0xffff; i = node_next(i))
      if (meta_id(node_meta(i)) == ip) return i;
    return -1;
  }
  // Links node i (already counted in nodeCount) into the hash; executed by one lane.
  BPSX_DEV void link(int i, uint32_t ip) const {
    const uint32_t b = hash(ip);
    const uint16_t head = L->first[b];
    if (i < kNodesLds) L->n_next[i] = head;
    else ws->next[i] = head;
    L->first[b] = (uint16_t)i;
  }

  // ---------------------------------------------------------------- open list
  BPSX_DEV HeapEntry hget(int i) const { return i < kHeapLds ? L->heap[i] : ws->heap_spill[i]; }
  BPSX_DEV float ht(int i) const { return hget(i).total; }
  BPSX_DEV int hn(int i) const { return (int)hget(i).node; }
  BPSX_DEV void hset(int i, float t, int n) const {
    const HeapEntry e{t, (uint32_t)n};
    if (i < kHeapLds) L->heap[i] = e;
    else ws->heap_spill[i] = e;
  }
  // dtNodeQueue::bubbleUp from index i0 with entry (t, n), all ancestors looked at at once:
  // along a leaf-to-root path the keys never increase, so the ancestors that are greater than
  // t form a prefix; they each move one level down and the entry lands above them.
  BPSX_DEV void bubble_up(int i0, float t, int n) const {
    // lane d holds ancestor a_d = ((i0 + 1) >> d) - 1 (a_0 = i0; -1 once past the root)
    const int a = lane <= 12 ? ((i0 + 1) >> lane) - 1 : -1;
    const bool valid = lane >= 1 && a >= 0;
    float at = 0;
    int an = 0;
    if (valid) { const HeapEntry e = hget(a); at = e.total; an = (int)e.node; }
    const unsigned long long gt = __ballot(valid && at > t);
    const int m = __popcll(gt);  // ancestors 1..m move down
    wave_sync();
    // lane d (1..m) writes its ancestor's entry one level down, into a_{d-1}
    const int child = lane >= 1 && lane <= 13 ? ((i0 + 1) >> (lane - 1)) - 1 : 0;
    if (lane >= 1 && lane <= m) hset(child, at, an);
    if (lane == m) hset(lane == 0 ? i0 : a, t, n);
    wave_sync();
  }
  BPSX_DEV void push(float t, int n) {
    heapSize++;
    bubble_up(heapSize - 1, t, n);
  }
  BPSX_DEV void modify(int n, float t) const {
    int found = -1;
    for (int base = 0; base < heapSize; base += 64) {
      const int i = base + lane;
      const unsigned long long m = __ballot(i < heapSize && hn(i) == n);
      if (m) { found = base + (__ffsll((long long)m) - 1); break; }
    }
    if (found >= 0) bubble_up(found, t, n);
  }
  // dtNodeQueue::pop: the hole left by the root travels down along the smaller children to a
  // leaf, then the former last entry bubbles up from there.  The route depends only on the
  // heap's contents, so lanes evaluate "which child is smaller" for 63 nodes of a subtree at
  // once and the route is then read off with scalar lane reads; the entries on the route that
  // are not greater than the re-inserted entry shift up one level, it lands below them, and
  // the rest of the route stays as it was.
  BPSX_DEV int pop() {
    const int top = hn(0);
    heapSize--;
    const int size = heapSize;
    if (size == 0) return top;
    const HeapEntry lastE = hget(size);
    const float lt = lastE.total;
    const int ln = (int)lastE.node;
    // route entries are collected one per lane: lane d keeps the d-th node of the route
    float myT = 0;
    int myN = 0, myIdx = -1, myParent = -1;
    int depth = 0;   // number of route nodes below the root found so far (uniform)
    int root = 0;    // root of the subtree being resolved (uniform)
    for (;;) {
      // lane t (< 63) looks at node (root+1 << lvl) - 1 + off of the subtree, lvl = floor(log2(t+1))
      const int t1 = lane + 1;
      const int lvl = 31 - __clz(t1);
      const int node = ((root + 1) << lvl) - 1 + (t1 - (1 << lvl));
      int choice = -1;
      float ct = 0;
      int cn = 0;
      if (lane < 63) {
        const int c1 = 2 * node + 1;
        if (c1 < size) {
          const HeapEntry e1 = hget(c1);
          ct = e1.total; cn = (int)e1.node; choice = c1;
          if (c1 + 1 < size) {
            const HeapEntry e2 = hget(c1 + 1);
            if (ct > e2.total) { ct = e2.total; cn = (int)e2.node; choice = c1 + 1; }
          }
        }
      }
      // follow the choices from the subtree's root: relative lane r -> 2r+1 or 2r+2
      int r = 0, cur = root;
      bool more = false;
      for (int s = 0; s < 6; ++s) {
        const int c = lane_i(choice, r);
        if (c < 0) break;
        const float tt = lane_f(ct, r);
        const int nn = lane_i(cn, r);
        depth++;
        if (lane == depth) { myT = tt; myN = nn; myIdx = c; myParent = cur; }
        r = 2 * r + 1 + (c - (2 * cur + 1));
        cur = c;
        if (r >= 63) { more = true; break; }
      }
      if (!more) break;
      root = cur;
    }
    const unsigned long long le = __ballot(lane >= 1 && lane <= depth && myT <= lt);
    const int j = __popcll(le);  // route entries 1..j shift up, the re-inserted entry lands at route[j]
    wave_sync();
    if (lane >= 1 && lane <= j) hset(myParent, myT, myN);
    if (lane == j) hset(j == 0 ? 0 : myIdx, lt, ln);
    wave_sync();
    return top;
  }
};

// Runs A* for one query. Returns the corridor length (corridor written to F->corridor), or 0
// when the reference would report anything but plain DT_SUCCESS.
BPSX_DEV int astar(GeoWave& g, FunnelLds* F, const NavData& nav, const SceneDev& s, uint32_t startIp, uint32_t endIp,
                   const float* startPos, const float* endPos, uint32_t* pops
#ifdef BPSX_PHASE_TIMING
                   , unsigned long long* phase_acc
#endif
                   ) {
  const int lane = g.lane;
#ifdef BPSX_PHASE_TIMING
  unsigned long long phase_t0 = __builtin_readcyclecounter();
#endif
  if (startIp == endIp) {
    if (lane == 0) F->corridor[0] = (uint16_t)startIp;
    wave_sync();
    return 1;
  }
  g.clear();
  const float H_SCALE = 0.999f;
  {
    const float dx = endPos[0] - startPos[0], dy = endPos[1] - startPos[1], dz = endPos[2] - startPos[2];
    const float total = sqrtf(dx * dx + dy * dy + dz * dz) * H_SCALE;
    g.nodeCount = 1;
    if (lane == 0) {
      NodeVal v;
      v.pos[0] = startPos[0]; v.pos[1] = startPos[1]; v.pos[2] = startPos[2];
      v.cost = 0; v.total = total; v.meta = meta_pack(startIp, 1u, 0u);
      g.node_store(0, v);
      g.link(0, startIp);
    }
    wave_sync();
    g.push(total, 0);
  }
  int lastBest = 0;
  float lastBestCost = g.L->n_total[0];
  bool outOfNodes = false;
  while (g.heapSize > 0) {
    // the node about to be popped is the root: fetch its polygon while the heap is repaired
    const int bi = uniform_i(g.hn(0));
    const NodeVal best = g.node_load(bi);
    const uint32_t bestIp = meta_id(best.meta);
    const PolyRec* bp = &nav.polys[s.poly_base + bestIp];
    uint32_t nbRaw = 0, nbWalk = 0;
    float l0 = 0, l1 = 0, l2 = 0, r0 = 0, r1 = 0, r2 = 0;
    const int nv = bp->nv;
    if (lane < kNvp) {
      nbRaw = bp->nei[lane];
      nbWalk = bp->walk[lane];
      l0 = bp->v[lane][0]; l1 = bp->v[lane][1]; l2 = bp->v[lane][2];
      if (lane + 1 < kNvp) { r0 = bp->v[lane + 1][0]; r1 = bp->v[lane + 1][1]; r2 = bp->v[lane + 1][2]; }
    }
    const uint32_t pidx = meta_pidx(best.meta);
    const uint32_t parentIp = pidx ? meta_id(g.node_meta((int)pidx - 1)) : kInvalidPoly;
    PHASE_MARK(0);
    g.pop();
    PHASE_MARK(1);
    if (lane == 0) g.node_set_meta(bi, meta_pack(bestIp, (meta_flags(best.meta) & ~1u) | 2u, pidx));
    wave_sync();
    if (bestIp == endIp) { lastBest = bi; break; }
    (*pops)++;
    // right end of edge j is vertex j+1, wrapping to vertex 0 on the last edge
    {
      const float w0 = lane_f(l0, 0), w1 = lane_f(l1, 0), w2 = lane_f(l2, 0);
      if (lane + 1 >= nv) { r0 = w0; r1 = w1; r2 = w2; }
    }
    // ---- per-edge phase: lane j looks at edge j
    uint32_t nb = kInvalidPoly;
    if (lane < nv) {
      const uint32_t w = (nbRaw & 0x8000u) ? 0u : nbRaw;
      if (w && (w - 1) != parentIp && nbWalk) nb = w - 1;
    }
    // a polygon reached through two edges of the same expansion: the second visit never
    // changes the node (same position, same cost), so only the first edge counts
    {
      const uint32_t orig = nb;
#pragma unroll
      for (int k = 0; k < kNvp - 1; ++k) {
        const uint32_t other = (uint32_t)lane_i((int)orig, k);
        if (lane > k && other == orig) nb = kInvalidPoly;
      }
    }
    PHASE_MARK(2);
    int ni = -1;
    if (nb != kInvalidPoly) ni = g.find(nb);
    PHASE_MARK(3);
    // new nodes take consecutive indices in edge order; past the pool's end they are dropped
    {
      const unsigned long long need = __ballot(nb != kInvalidPoly && ni < 0);
      if (need) {
        const int rank = __popcll(need & ((1ull << lane) - 1ull));
        const bool mine = (need >> lane) & 1ull;
        if (mine) {
          const int idx = g.nodeCount + rank;
          if (idx < kMaxNodes) ni = idx;
          else nb = kInvalidPoly;
        }
        const int want = g.nodeCount + __popcll(need);
        if (want > kMaxNodes) outOfNodes = true;
        g.nodeCount = want < kMaxNodes ? want : kMaxNodes;
        // hash insertion one node at a time (two new nodes may share a bucket)
        unsigned long long todo = need;
        while (todo) {
          const int src = __ffsll((long long)todo) - 1;
          todo &= todo - 1;
          if (lane == src && nb != kInvalidPoly) g.link(ni, nb);
          wave_sync();
        }
        if (mine && nb != kInvalidPoly) {
          NodeVal v;
          v.pos[0] = v.pos[1] = v.pos[2] = 0; v.cost = 0; v.total = 0; v.meta = meta_pack(nb, 0u, 0u);
          g.node_store(ni, v);
        }
      }
    }
    PHASE_MARK(4);
    bool update = false;
    float total = 0, heuristic = 0;
    bool wasOpen = false;
    if (nb != kInvalidPoly) {
      NodeVal nn = g.node_load(ni);
      uint32_t fl = meta_flags(nn.meta);
      if (fl == 0) {
        nn.pos[0] = (l0 + r0) * 0.5f;
        nn.pos[1] = (l1 + r1) * 0.5f;
        nn.pos[2] = (l2 + r2) * 0.5f;
      }
      const float cx = nn.pos[0] - best.pos[0], cy = nn.pos[1] - best.pos[1], cz = nn.pos[2] - best.pos[2];
      const float curCost = sqrtf(cx * cx + cy * cy + cz * cz) * 1.0f;
      const float ex = endPos[0] - nn.pos[0], ey = endPos[1] - nn.pos[1], ez = endPos[2] - nn.pos[2];
      const float toEnd = sqrtf(ex * ex + ey * ey + ez * ez);
      float cost;
      if (nb == endIp) {
        cost = best.cost + curCost + toEnd * 1.0f;
        heuristic = 0;
      } else {
        cost = best.cost + curCost;
        heuristic = toEnd * H_SCALE;
      }
      total = cost + heuristic;
      const bool worse = (fl & 3u) && total >= nn.total;
      if (!worse) {
        update = true;
        wasOpen = (fl & 1u) != 0;
        nn.meta = meta_pack(nb, (fl & ~2u) | 1u, (uint32_t)bi + 1);
        nn.cost = cost;
        nn.total = total;
        g.node_store(ni, nn);
      }
    }
    wave_sync();
    PHASE_MARK(5);
    // ---- ordered phase: heap and "nearest so far" updates in edge order
    unsigned long long upd = __ballot(update);
    while (upd) {
      const int src = __ffsll((long long)upd) - 1;
      upd &= upd - 1;
      const int node = lane_i(ni, src);
      const float t = lane_f(total, src);
      const float h = lane_f(heuristic, src);
      const bool open = lane_i(wasOpen ? 1 : 0, src) != 0;
      if (open) g.modify(node, t);
      else g.push(t, node);
      if (h < lastBestCost) { lastBestCost = h; lastBest = node; }
    }
    PHASE_MARK(6);
  }
  // getPathToNode
  int length = 0;
  for (int c = lastBest + 1; c; c = (int)meta_pidx(g.node_meta(c - 1))) length++;
  const bool ok = length <= kMaxPath && meta_id(g.node_meta(lastBest)) == endIp && !outOfNodes;
  if (!ok) return 0;
  // the corridor goes into LDS that overlays the nodes' cost and position arrays; the parent
  // links (n_meta) are outside that region and stay readable while it is written
  if (lane == 0) {
    int c = lastBest + 1;
    for (int i = length - 1; i >= 0; --i) {
      const uint32_t m = g.node_meta(c - 1);
      F->corridor[i] = (uint16_t)meta_id(m);
      c = (int)meta_pidx(m);
    }
  }
  wave_sync();
  return length;
}

BPSX_DEV float tri_area2d(const float* a, const float* b, const float* c) {
  const float abx = b[0] - a[0], abz = b[2] - a[2];
  const float acx = c[0] - a[0], acz = c[2] - a[2];
  return acx * abz - abx * acz;
}
BPSX_DEV bool vequal(const float* a, const float* b) {
  const float thr = (1.0f / 16384.0f) * (1.0f / 16384.0f);
  const float dx = b[0] - a[0], dy = b[1] - a[1], dz = b[2] - a[2];
  return dx * dx + dy * dy + dz * dz < thr;
}

// String pulling over F->corridor[0..n) and the summed length; +inf for every outcome the
// reference maps to "no path" (straight path of 256 points or more, missing portal).
BPSX_DEV float funnel_length(int lane, FunnelLds* F, const NavData& nav, const SceneDev& s, int n, const float* startPos,
                             const float* endPos) {
  const float INF = __int_as_float(0x7f800000);
  // gather the portals of the corridor, 64 at a time
  bool missing = false;
  for (int i = lane; i + 1 < n; i += 64) {
    const PolyRec& r = nav.polys[s.poly_base + F->corridor[i]];
    const uint32_t to = F->corridor[i + 1];
    int e = -1;
    for (int k = 0; k < r.nv; ++k)
      if (r.nei[k] && !(r.nei[k] & 0x8000) && (uint32_t)(r.nei[k] - 1) == to) { e = k; break; }
    if (e < 0) { missing = true; continue; }
    const float* l = r.v[e];
    const float* rr = r.v[(e + 1) % r.nv];
    float* p = F->portals[i];
    p[0] = l[0]; p[1] = l[1]; p[2] = l[2]; p[3] = rr[0]; p[4] = rr[1]; p[5] = rr[2];
  }
  wave_sync();
  if (__ballot(missing)) return INF;
  float cs[3], ce[3];
  closest_on_poly_boundary(nav.polys[s.poly_base + F->corridor[0]], startPos, cs);
  closest_on_poly_boundary(nav.polys[s.poly_base + F->corridor[n - 1]], endPos, ce);
  // straight-path points are only needed pairwise: keep the last one and the running length
  float last[3] = {cs[0], cs[1], cs[2]};
  int npts = 1;
  float length = 0.0f;
  bool finished = false, overflow = false;
  auto append = [&](const float* p, bool isEnd) {
    if (vequal(last, p)) return;  // merged with the previous point
    const float dx = last[0] - p[0], dy = last[1] - p[1], dz = last[2] - p[2];
    length += sqrtf(dx * dx + (dy * dy + dz * dz));
    last[0] = p[0]; last[1] = p[1]; last[2] = p[2];
    npts++;
    if (npts >= kMaxPath) { overflow = true; finished = true; return; }
    if (isEnd) finished = true;
  };
  if (n > 1) {
    float apex[3] = {cs[0], cs[1], cs[2]}, pl[3] = {cs[0], cs[1], cs[2]}, pr[3] = {cs[0], cs[1], cs[2]};
    int apexIndex = 0, leftIndex = 0, rightIndex = 0;
    bool leftIsEnd = false, rightIsEnd = false;  // "poly ref == 0" of the reference
    for (int i = 0; i < n && !finished; ++i) {
      float left[3], right[3];
      if (i + 1 < n) {
        const float* p = F->portals[i];
        left[0] = p[0]; left[1] = p[1]; left[2] = p[2];
        right[0] = p[3]; right[1] = p[4]; right[2] = p[5];
        if (i == 0) {
          float t;
          if (dist_pt_seg_sqr2d(apex[0], apex[2], left, right, t) < 0.001f * 0.001f) continue;
        }
      } else {
        left[0] = right[0] = ce[0]; left[1] = right[1] = ce[1]; left[2] = right[2] = ce[2];
      }
      if (tri_area2d(apex, pr, right) <= 0.0f) {
        if (vequal(apex, pr) || tri_area2d(apex, pl, right) > 0.0f) {
          pr[0] = right[0]; pr[1] = right[1]; pr[2] = right[2];
          rightIsEnd = !(i + 1 < n);
          rightIndex = i;
        } else {
          apex[0] = pl[0]; apex[1] = pl[1]; apex[2] = pl[2];
          apexIndex = leftIndex;
          append(apex, leftIsEnd);
          if (finished) break;
          pl[0] = pr[0] = apex[0]; pl[1] = pr[1] = apex[1]; pl[2] = pr[2] = apex[2];
          leftIndex = rightIndex = apexIndex;
          i = apexIndex;
          continue;
        }
      }
      if (tri_area2d(apex, pl, left) >= 0.0f) {
        if (vequal(apex, pl) || tri_area2d(apex, pr, left) < 0.0f) {
          pl[0] = left[0]; pl[1] = left[1]; pl[2] = left[2];
          leftIsEnd = !(i + 1 < n);
          leftIndex = i;
        } else {
          apex[0] = pr[0]; apex[1] = pr[1]; apex[2] = pr[2];
          apexIndex = rightIndex;
          append(apex, rightIsEnd);
          if (finished) break;
          pl[0] = pr[0] = apex[0]; pl[1] = pr[1] = apex[1]; pl[2] = pr[2] = apex[2];
          leftIndex = rightIndex = apexIndex;
          i = apexIndex;
          continue;
        }
      }
    }
  }
  if (!finished) {
    append(ce, true);
    if (npts >= kMaxPath) overflow = true;
  }
  return overflow ? INF : length;
}

// Full PathFinder::findPath distance for one query, executed by a wavefront.
BPSX_DEV float geodesic_query(GeoWave& g, const NavData& nav, const GeoQuery& q, uint32_t* pops, uint32_t* corridor
#ifdef BPSX_PHASE_TIMING
                              , unsigned long long* phase_acc
#endif
                              ) {
  const float INF = __int_as_float(0x7f800000);
  {
    // Eigen isApprox with default precision; sums of three reduce as a0 + (a1 + a2)
    const float d0 = q.a[0] - q.b[0], d1 = q.a[1] - q.b[1], d2 = q.a[2] - q.b[2];
    const float dd = d0 * d0 + (d1 * d1 + d2 * d2);
    const float aa = q.a[0] * q.a[0] + (q.a[1] * q.a[1] + q.a[2] * q.a[2]);
    const float bb = q.b[0] * q.b[0] + (q.b[1] * q.b[1] + q.b[2] * q.b[2]);
    const float mn = bb < aa ? bb : aa;
    const float prec = 1e-5f;
    if (dd <= prec * prec * mn) return 0.0f;
  }
  const SceneDev& s = nav.scenes[q.scene];
  const uint32_t sIp = decode_ref(s, q.a_ref), eIp = decode_ref(s, q.b_ref);
  if (sIp == kInvalidPoly || eIp == kInvalidPoly) return INF;
  if (nav.polys[s.poly_base + sIp].island != nav.polys[s.poly_base + eIp].island) return INF;
  if (!finite3(q.a[0], q.a[1], q.a[2]) || !finite3(q.b[0], q.b[1], q.b[2])) return INF;
  FunnelLds* F = reinterpret_cast<FunnelLds*>(g.L);
#ifdef BPSX_PHASE_TIMING
  const int n = astar(g, F, nav, s, sIp, eIp, q.a, q.b, pops, phase_acc);
  unsigned long long phase_t0 = __builtin_readcyclecounter();
#else
  const int n = astar(g, F, nav, s, sIp, eIp, q.a, q.b, pops);
#endif
  if (n <= 0) return INF;
  *corridor += (uint32_t)n;
  const float len = funnel_length(g.lane, F, nav, s, n, q.a, q.b);
  PHASE_MARK(7);
  return len;
}

}  // namespace bpsx
