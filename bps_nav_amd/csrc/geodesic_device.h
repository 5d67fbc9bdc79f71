// Geodesic distance on the GPU: Detour's A* over the polygon graph followed by the funnel
// (string pulling) and the summed segment length, with the exact buffer limits and failure
// conventions of the reference, so that the value equals PathFinder::findPath's.
//
// Execution model: a group of G consecutive lanes of one wavefront (G = 8, 16, 32 or 64)
// owns one query at a time and pulls the next from a shared queue when done.  Inside a
// group the sequential parts of A* (heap, node allocation order, funnel) run redundantly on
// all lanes with lane 0 doing the stores; the per-edge work of a node expansion (neighbour
// lookup in the node pool, portal midpoint, cost) is spread over the lanes.
// The open list's top levels and the hash heads live in LDS, the node pool in a per-slot
// scratch area in HBM.
//
// Reference semantics followed: DetourNavMeshQuery.cpp:945-1178 (findPath, getPathToNode),
// :1661-1696, 1765-1994 (appendVertex, findStraightPath), :2279-2349 (getPortalPoints);
// DetourNode.cpp:50-200 (node pool, heap order); PathFinder.cpp:473-541.
#pragma once
#include "nav_device.h"

namespace bpsx {

constexpr int kHeapLds = 256;   // open-list entries kept in LDS per group
constexpr int kHashSize = 512;

BPSX_DEV void group_sync() {
  // Lanes of a group share a wavefront: ordering only has to be imposed on the compiler.
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

template <int G>
BPSX_DEV uint32_t group_ballot(bool p, int grp) {
  const unsigned long long m = __ballot(p);
  if (G == 64) return 0;  // not used with 64 (callers use the 64-bit form)
  return (uint32_t)((m >> (grp * G)) & ((1ull << G) - 1ull));
}

template <int G>
struct GeoGroup {
  HeapEntry* heap_lds;   // [kHeapLds]
  uint16_t* first;       // [kHashSize]
  GeoSlot* ws;
  int lane;              // 0..G-1
  int grp;               // group index within the wavefront
  int heapSize;
  int nodeCount;

  BPSX_DEV unsigned long long gballot(bool p) const {
    const unsigned long long m = __ballot(p);
    if (G == 64) return m;
    return (m >> (grp * G)) & ((1ull << G) - 1ull);
  }
  BPSX_DEV HeapEntry hget(int i) const { return i < kHeapLds ? heap_lds[i] : ws->heap_spill[i]; }
  BPSX_DEV void hset(int i, HeapEntry e) const {
    if (lane == 0) {
      if (i < kHeapLds) heap_lds[i] = e;
      else ws->heap_spill[i] = e;
    }
  }
  BPSX_DEV void bubble_up(int i, HeapEntry e) const {
    int parent = (i - 1) / 2;
    while (i > 0) {
      const HeapEntry pe = hget(parent);
      if (!(pe.total > e.total)) break;
      hset(i, pe);
      i = parent;
      parent = (i - 1) / 2;
    }
    hset(i, e);
    group_sync();
  }
  BPSX_DEV void trickle_down(int i, HeapEntry e) const {
    int child = i * 2 + 1;
    while (child < heapSize) {
      HeapEntry c = hget(child);
      if (child + 1 < heapSize) {
        const HeapEntry c2 = hget(child + 1);
        if (c.total > c2.total) { child++; c = c2; }
      }
      hset(i, c);
      i = child;
      child = i * 2 + 1;
    }
    group_sync();
    bubble_up(i, e);
  }
  BPSX_DEV void push(HeapEntry e) {
    heapSize++;
    bubble_up(heapSize - 1, e);
  }
  BPSX_DEV HeapEntry pop() {
    const HeapEntry r = hget(0);
    heapSize--;
    const HeapEntry last = hget(heapSize);
    group_sync();
    trickle_down(0, last);
    return r;
  }
  // dtNodeQueue::modify: locate the node's entry (lanes scan in parallel), give it its new
  // key and bubble it up from where it was.
  BPSX_DEV void modify(uint32_t node, float total) const {
    int found = -1;
    for (int base = 0; base < heapSize; base += G) {
      const int i = base + lane;
      const bool hit = i < heapSize && hget(i).node == node;
      const unsigned long long m = gballot(hit);
      if (m) { found = base + (__ffsll((long long)m) - 1); break; }
    }
    if (found >= 0) bubble_up(found, HeapEntry{total, node});
  }
  static BPSX_DEV uint32_t hash(uint32_t a) {
    a ^= a >> 16; a *= 0x7feb352du; a ^= a >> 15; a *= 0x846ca68bu; a ^= a >> 16;
    return a & (kHashSize - 1);
  }
  BPSX_DEV void clear() {
    for (int i = lane; i < kHashSize; i += G) first[i] = 0xffff;
    heapSize = 0;
    nodeCount = 0;
    group_sync();
  }
  // node index of polygon `ip`, or -1
  BPSX_DEV int find(uint32_t ip) const {
    for (uint32_t i = first[hash(ip)]; i != 0xffff; i = ws->next[i])
      if (ws->nodes[i].id == ip) return (int)i;
    return -1;
  }
  // Appends a node for `ip` (lane 0 writes); returns its index or -1 when the pool is full.
  BPSX_DEV int alloc(uint32_t ip) {
    if (nodeCount >= kMaxNodes) return -1;
    const int i = nodeCount++;
    const uint32_t b = hash(ip);
    if (lane == 0) {
      ws->next[i] = first[b];
      first[b] = (uint16_t)i;
      ANode& n = ws->nodes[i];
      n.pidx = 0; n.cost = 0; n.total = 0; n.id = ip; n.flags = 0;
    }
    group_sync();
    return i;
  }
};

template <int G>
BPSX_DEV float bcast_f(float v, int src) { return __shfl(v, src, G); }
template <int G>
BPSX_DEV int bcast_i(int v, int src) { return __shfl(v, src, G); }

// Runs A* for one query. Returns the corridor length written to ws->corridor, or 0 when the
// reference would report anything but plain DT_SUCCESS.
template <int G>
BPSX_DEV int astar(GeoGroup<G>& g, const NavData& nav, const SceneDev& s, uint32_t startIp, uint32_t endIp,
                   const float* startPos, const float* endPos, uint32_t* pops) {
  const int lane = g.lane;
  GeoSlot* ws = g.ws;
  if (startIp == endIp) {
    if (lane == 0) ws->corridor[0] = startIp;
    group_sync();
    return 1;
  }
  g.clear();
  const float H_SCALE = 0.999f;
  {
    const int si = g.alloc(startIp);
    const float dx = endPos[0] - startPos[0], dy = endPos[1] - startPos[1], dz = endPos[2] - startPos[2];
    const float total = sqrtf(dx * dx + dy * dy + dz * dz) * H_SCALE;
    if (lane == 0) {
      ANode& n = ws->nodes[si];
      n.pos[0] = startPos[0]; n.pos[1] = startPos[1]; n.pos[2] = startPos[2];
      n.pidx = 0; n.cost = 0; n.total = total; n.id = startIp; n.flags = 1;
    }
    group_sync();
    g.push(HeapEntry{total, (uint32_t)si});
  }
  int lastBest = 0;
  float lastBestCost = ws->nodes[0].total;
  bool outOfNodes = false;
  while (g.heapSize > 0) {
    const HeapEntry top = g.pop();
    const int bi = (int)top.node;
    const ANode best = ws->nodes[bi];
    if (lane == 0) ws->nodes[bi].flags = (best.flags & ~1u) | 2u;
    group_sync();
    if (best.id == endIp) { lastBest = bi; break; }
    (*pops)++;
    const PolyRec& bp = nav.polys[s.poly_base + best.id];
    const uint32_t parentIp = best.pidx ? ws->nodes[best.pidx - 1].id : kInvalidPoly;
    // ---- per-edge phase: lane j looks at edge j
    const int nv = bp.nv;
    uint32_t nb = kInvalidPoly;
    if (lane < nv) {
      const uint16_t w = (bp.nei[lane] & 0x8000) ? (uint16_t)0 : bp.nei[lane];
      // the link exists for every internal edge; the filter is applied to the neighbour
      if (w && (uint32_t)(w - 1) != parentIp && bp.walk[lane]) nb = (uint32_t)(w - 1);
    }
    // a polygon reached through two edges of the same expansion: the second visit never
    // changes the node (same position, same cost), so only the first edge counts
    for (int k = 0; k < kNvp - 1; ++k) {
      const uint32_t other = (uint32_t)bcast_i<G>((int)nb, k);
      if (lane > k && nb != kInvalidPoly && other == nb) nb = kInvalidPoly;
    }
    int ni = -1;
    if (nb != kInvalidPoly) ni = g.find(nb);
    // allocation in edge order (the pool may run out part-way)
    unsigned long long need = g.gballot(nb != kInvalidPoly && ni < 0);
    while (need) {
      const int src = __ffsll((long long)need) - 1;
      need &= need - 1;
      const uint32_t ip = (uint32_t)bcast_i<G>((int)nb, src);
      const int idx = g.alloc(ip);
      if (idx < 0) outOfNodes = true;
      if (lane == src) { ni = idx; if (idx < 0) nb = kInvalidPoly; }
    }
    bool update = false;
    float total = 0, heuristic = 0;
    bool wasOpen = false;
    if (nb != kInvalidPoly) {
      ANode nn = ws->nodes[ni];
      if (nn.flags == 0) {
        const float* l = bp.v[lane];
        const float* r = bp.v[(lane + 1) % nv];
        nn.pos[0] = (l[0] + r[0]) * 0.5f;
        nn.pos[1] = (l[1] + r[1]) * 0.5f;
        nn.pos[2] = (l[2] + r[2]) * 0.5f;
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
      const bool worse = (nn.flags & 3u) && total >= nn.total;
      if (!worse) {
        update = true;
        wasOpen = (nn.flags & 1u) != 0;
        nn.pidx = (uint32_t)bi + 1;
        nn.id = nb;
        nn.flags = (nn.flags & ~2u) | 1u;
        nn.cost = cost;
        nn.total = total;
        ws->nodes[ni] = nn;
      }
    }
    group_sync();
    // ---- ordered phase: heap and "nearest so far" updates in edge order
    unsigned long long upd = g.gballot(update);
    while (upd) {
      const int src = __ffsll((long long)upd) - 1;
      upd &= upd - 1;
      const int node = bcast_i<G>(ni, src);
      const float t = bcast_f<G>(total, src);
      const float h = bcast_f<G>(heuristic, src);
      const bool open = bcast_i<G>(wasOpen ? 1 : 0, src) != 0;
      if (open) g.modify((uint32_t)node, t);
      else g.push(HeapEntry{t, (uint32_t)node});
      if (h < lastBestCost) { lastBestCost = h; lastBest = node; }
    }
  }
  // getPathToNode
  int length = 0;
  for (int c = lastBest + 1; c; c = (int)ws->nodes[c - 1].pidx) length++;
  const bool ok = length <= kMaxPath && ws->nodes[lastBest].id == endIp && !outOfNodes;
  if (!ok) return 0;
  if (lane == 0) {
    int c = lastBest + 1;
    for (int i = length - 1; i >= 0; --i) {
      ws->corridor[i] = ws->nodes[c - 1].id;
      c = (int)ws->nodes[c - 1].pidx;
    }
  }
  group_sync();
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

// String pulling over ws->corridor[0..n) and the summed length; +inf for every outcome the
// reference maps to "no path" (straight path of 256 points or more, missing portal).
template <int G>
BPSX_DEV float funnel_length(GeoGroup<G>& g, const NavData& nav, const SceneDev& s, int n, const float* startPos,
                             const float* endPos) {
  GeoSlot* ws = g.ws;
  const float INF = __int_as_float(0x7f800000);
  // gather the portals of the corridor, G at a time
  bool missing = false;
  for (int i = g.lane; i + 1 < n; i += G) {
    const PolyRec& r = nav.polys[s.poly_base + ws->corridor[i]];
    const uint32_t to = ws->corridor[i + 1];
    int e = -1;
    for (int k = 0; k < r.nv; ++k)
      if (r.nei[k] && !(r.nei[k] & 0x8000) && (uint32_t)(r.nei[k] - 1) == to) { e = k; break; }
    if (e < 0) { missing = true; continue; }
    const float* l = r.v[e];
    const float* rr = r.v[(e + 1) % r.nv];
    float* p = ws->portals[i];
    p[0] = l[0]; p[1] = l[1]; p[2] = l[2]; p[3] = rr[0]; p[4] = rr[1]; p[5] = rr[2];
  }
  group_sync();
  if (g.gballot(missing)) return INF;
  float cs[3], ce[3];
  closest_on_poly_boundary(nav.polys[s.poly_base + ws->corridor[0]], startPos, cs);
  closest_on_poly_boundary(nav.polys[s.poly_base + ws->corridor[n - 1]], endPos, ce);
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
        const float* p = ws->portals[i];
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

// Full PathFinder::findPath distance for one query, executed by a group.
template <int G>
BPSX_DEV float geodesic_query(GeoGroup<G>& g, const NavData& nav, const GeoQuery& q, uint32_t* pops, uint32_t* corridor) {
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
  const int n = astar<G>(g, nav, s, sIp, eIp, q.a, q.b, pops);
  if (n <= 0) return INF;
  *corridor += (uint32_t)n;
  return funnel_length<G>(g, nav, s, n, q.a, q.b);
}

}  // namespace bpsx
