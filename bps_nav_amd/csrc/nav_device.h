// Device-side navmesh queries on PolyRec records: the geometry primitives and the
// per-lane queries (nearest polygon, move along surface, height) of the step path.
// Compile with -ffp-contract=off: polygon ids must equal the reference's bit for bit, so
// every expression keeps Detour's fp32 operation order and is never fused.
//
// Reference semantics followed (read, not copied):
//   DetourCommon.cpp:170-184 (point-segment distance), :204-233 (height on triangle),
//   :238-270 (point in polygon, edge distances), :332-369 (random point in polygon);
//   DetourNavMesh.cpp:619-758 (height mesh queries); DetourNavMeshQuery.cpp:538-586
//   (boundary clamp), :642-826 (nearest polygon over the BV tree), :2016-2255 (move along
//   surface); PathFinder.cpp:24-44, 543-584 (snapPoint / tryStep conventions).
#pragma once
#include <hip/hip_runtime.h>

#include "device_types.h"

namespace bpsx {

#define BPSX_DEV __device__ __forceinline__

struct NavPt {
  float x, y, z;
  uint32_t ref;
};

BPSX_DEV bool finite3(float x, float y, float z) { return isfinite(x) && isfinite(y) && isfinite(z); }

BPSX_DEV float dist_pt_seg_sqr2d(float px, float pz, const float* p, const float* q, float& t) {
  const float pqx = q[0] - p[0], pqz = q[2] - p[2];
  float dx = px - p[0], dz = pz - p[2];
  const float d = pqx * pqx + pqz * pqz;
  t = pqx * dx + pqz * dz;
  if (d > 0) t /= d;
  if (t < 0) t = 0;
  else if (t > 1) t = 1;
  dx = p[0] + t * pqx - px;
  dz = p[2] + t * pqz - pz;
  return dx * dx + dz * dz;
}

BPSX_DEV bool point_in_poly(float px, float pz, const PolyRec& r) {
  bool c = false;
  const int nv = r.nv;
  for (int i = 0, j = nv - 1; i < nv; j = i++) {
    const float* vi = r.v[i];
    const float* vj = r.v[j];
    if (((vi[2] > pz) != (vj[2] > pz)) && (px < (vj[0] - vi[0]) * (pz - vi[2]) / (vj[2] - vi[2]) + vi[0])) c = !c;
  }
  return c;
}

BPSX_DEV bool height_on_triangle(float px, float pz, const float* a, const float* b, const float* c, float& h) {
  const float EPS = 1e-6f;
  const float v0x = c[0] - a[0], v0y = c[1] - a[1], v0z = c[2] - a[2];
  const float v1x = b[0] - a[0], v1y = b[1] - a[1], v1z = b[2] - a[2];
  const float v2x = px - a[0], v2z = pz - a[2];
  float denom = v0x * v1z - v0z * v1x;
  if (fabsf(denom) < EPS) return false;
  float u = v1z * v2x - v1x * v2z;
  float v = v0x * v2z - v0z * v2x;
  if (denom < 0) { denom = -denom; u = -u; v = -v; }
  if (u >= 0.0f && v >= 0.0f && (u + v) <= denom) {
    h = a[1] + (v0y * u + v1y * v) / denom;
    return true;
  }
  return false;
}

BPSX_DEV const float* detail_vert(const NavData& nav, const PolyRec& r, int k) {
  return k < r.nv ? r.v[k] : &nav.dverts[(size_t)(r.dvert_base + (uint32_t)(k - r.nv)) * 3];
}

template <bool kOnlyBoundary>
BPSX_DEV void closest_on_detail_edges(const NavData& nav, const PolyRec& r, float px, float py, float pz, float* out) {
  float dmin = 3.402823466e+38f, tmin = 0;
  const float* pmin = nullptr;
  const float* pmax = nullptr;
  for (int i = 0; i < r.tri_count; ++i) {
    const uint8_t* tris = &nav.dtris[(size_t)(r.tri_base + i) * 4];
    const uint8_t tf = tris[3];
    if (kOnlyBoundary && (tf & 0x15) == 0) continue;
    const float* v[3] = {detail_vert(nav, r, tris[0]), detail_vert(nav, r, tris[1]), detail_vert(nav, r, tris[2])};
    for (int k = 0, j = 2; k < 3; j = k++) {
      if ((((tf >> (j * 2)) & 1) == 0) && (kOnlyBoundary || tris[j] < tris[k])) continue;
      float t;
      const float d = dist_pt_seg_sqr2d(px, pz, v[j], v[k], t);
      if (d < dmin) { dmin = d; tmin = t; pmin = v[j]; pmax = v[k]; }
    }
  }
  if (!pmin) { out[0] = px; out[1] = py; out[2] = pz; return; }
  out[0] = pmin[0] + (pmax[0] - pmin[0]) * tmin;
  out[1] = pmin[1] + (pmax[1] - pmin[1]) * tmin;
  out[2] = pmin[2] + (pmax[2] - pmin[2]) * tmin;
}

// dtNavMesh::getPolyHeight: false when (px,pz) is outside the polygon.
BPSX_DEV bool poly_height(const NavData& nav, const PolyRec& r, float px, float py, float pz, float& h) {
  if (r.type != 0) return false;
  if (!point_in_poly(px, pz, r)) return false;
  for (int j = 0; j < r.tri_count; ++j) {
    const uint8_t* t = &nav.dtris[(size_t)(r.tri_base + j) * 4];
    if (height_on_triangle(px, pz, detail_vert(nav, r, t[0]), detail_vert(nav, r, t[1]), detail_vert(nav, r, t[2]), h))
      return true;
  }
  float c[3];
  closest_on_detail_edges<false>(nav, r, px, py, pz, c);
  h = c[1];
  return true;
}

// closestPointOnPolyBoundary: the point itself when inside (xz), else its projection onto
// the nearest polygon edge.
BPSX_DEV void closest_on_poly_boundary(const PolyRec& r, const float* pos, float* out) {
  float ed[kNvp], et[kNvp];
  bool c = false;
  const int nv = r.nv;
  for (int i = 0, j = nv - 1; i < nv; j = i++) {
    const float* vi = r.v[i];
    const float* vj = r.v[j];
    if (((vi[2] > pos[2]) != (vj[2] > pos[2])) &&
        (pos[0] < (vj[0] - vi[0]) * (pos[2] - vi[2]) / (vj[2] - vi[2]) + vi[0]))
      c = !c;
    ed[j] = dist_pt_seg_sqr2d(pos[0], pos[2], vj, vi, et[j]);
  }
  if (c) { out[0] = pos[0]; out[1] = pos[1]; out[2] = pos[2]; return; }
  float dmin = ed[0];
  int imin = 0;
  for (int i = 1; i < nv; ++i)
    if (ed[i] < dmin) { dmin = ed[i]; imin = i; }
  const float* va = r.v[imin];
  const float* vb = r.v[(imin + 1) % nv];
  const float t = et[imin];
  out[0] = va[0] + (vb[0] - va[0]) * t;
  out[1] = va[1] + (vb[1] - va[1]) * t;
  out[2] = va[2] + (vb[2] - va[2]) * t;
}

// Polygon index of a ref within its scene, or kInvalidPoly (dtNavMesh::isValidPolyRef).
BPSX_DEV uint32_t decode_ref(const SceneDev& s, uint32_t ref) {
  if (!ref) return kInvalidPoly;
  const uint32_t ip = ref & s.poly_mask;
  if ((ref & ~s.poly_mask) != s.ref_base || ip >= s.poly_count) return kInvalidPoly;
  return ip;
}

// One candidate of the nearest-polygon search: distance rule of dtFindNearestPolyQuery.
BPSX_DEV float snap_candidate(const NavData& nav, const SceneDev& s, const PolyRec& r, float px, float py, float pz,
                              float* cp) {
  float h;
  if (poly_height(nav, r, px, py, pz, h)) {
    cp[0] = px; cp[1] = h; cp[2] = pz;
    float d = fabsf(py - h) - s.climb;
    return d > 0 ? d * d : 0;
  }
  closest_on_detail_edges<true>(nav, r, px, py, pz, cp);
  const float dx = px - cp[0], dy = py - cp[1], dz = pz - cp[2];
  return dx * dx + dy * dy + dz * dz;
}

struct SnapBox {
  uint16_t bmin[3], bmax[3];
  bool hit_tile;
};
BPSX_DEV float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }
BPSX_DEV SnapBox snap_box(const SceneDev& s, float px, float py, float pz) {
  SnapBox b;
  const float qmin[3] = {px - 2.0f, py - 4.0f, pz - 2.0f};
  const float qmax[3] = {px + 2.0f, py + 4.0f, pz + 2.0f};
  const int minx = (int)floorf((qmin[0] - s.orig[0]) / s.tile_w), miny = (int)floorf((qmin[2] - s.orig[2]) / s.tile_h);
  const int maxx = (int)floorf((qmax[0] - s.orig[0]) / s.tile_w), maxy = (int)floorf((qmax[2] - s.orig[2]) / s.tile_h);
  b.hit_tile = !(s.tx < minx || s.tx > maxx || s.ty < miny || s.ty > maxy);
  for (int k = 0; k < 3; ++k) {
    const float lo = clampf(qmin[k], s.bmin[k], s.bmax[k]) - s.bmin[k];
    const float hi = clampf(qmax[k], s.bmin[k], s.bmax[k]) - s.bmin[k];
    b.bmin[k] = (uint16_t)((uint16_t)(int)(s.qfac * lo) & 0xfffe);
    b.bmax[k] = (uint16_t)((uint16_t)(int)(s.qfac * hi + 1) | 1);
  }
  return b;
}

// snapPoint, one lane per point: BV-tree walk with escape indices, candidates taken in tree
// order with a strict '<' so the first of equally near polygons wins.
BPSX_DEV NavPt snap_point(const NavData& nav, const SceneDev& s, float px, float py, float pz, uint32_t* ncand) {
  const float qnan = __int_as_float(0x7fc00000);
  NavPt out{qnan, qnan, qnan, 0};
  if (!finite3(px, py, pz)) return out;
  const SnapBox box = snap_box(s, px, py, pz);
  if (!box.hit_tile) return out;
  float best = 3.402823466e+38f;
  float bp[3] = {0, 0, 0};
  uint32_t bestIp = kInvalidPoly;
  uint32_t i = 0;
  while (i < s.bv_count) {
    const BVNodeDev nd = nav.bv[s.bv_base + i];
    bool overlap = true;
#pragma unroll
    for (int k = 0; k < 3; ++k)
      if (box.bmin[k] > nd.bmax[k] || box.bmax[k] < nd.bmin[k]) overlap = false;
    const bool leaf = nd.b == kBVLeaf;
    if (leaf && overlap) {
      const PolyRec& r = nav.polys[s.poly_base + (uint32_t)nd.a];
      if (r.flags & 1) {
        float cp[3];
        const float d = snap_candidate(nav, s, r, px, py, pz, cp);
        (*ncand)++;
        if (d < best) { best = d; bestIp = (uint32_t)nd.a; bp[0] = cp[0]; bp[1] = cp[1]; bp[2] = cp[2]; }
      }
    }
    if (overlap || leaf) i++;
    else i += (uint32_t)nd.a;
  }
  if (bestIp == kInvalidPoly || isnan(bp[0])) return out;
  out.x = bp[0]; out.y = bp[1]; out.z = bp[2];
  out.ref = s.ref_base | bestIp;
  return out;
}

// snapPoint by a whole wavefront (64 lanes), for callers where few points are snapped at a
// time.  The BV tree is descended level by level through an LDS frontier (every lane tests
// one node per round), the leaves that overlap the query box become candidates, each lane
// evaluates one candidate, and the winner is the smallest (distance, position in the tree's
// node array): the same polygon the in-order walk with its strict '<' picks.
constexpr int kSnapFrontier = 1024;
struct SnapLds {
  uint16_t frontier[2][kSnapFrontier];
  uint16_t cand_node[64];   // tree position of the candidates of the current batch
  uint16_t cand_poly[64];
};
BPSX_DEV NavPt snap_point_wave(const NavData& nav, const SceneDev& s, float px, float py, float pz, SnapLds& L,
                               uint32_t* ncand) {
  const int lane = (int)(threadIdx.x & 63);
  const float qnan = __int_as_float(0x7fc00000);
  NavPt out{qnan, qnan, qnan, 0};
  if (!finite3(px, py, pz)) return out;
  const SnapBox box = snap_box(s, px, py, pz);
  if (!box.hit_tile || s.bv_count == 0) return out;
  if (!s.bv_tree_ok) return snap_point(nav, s, px, py, pz, ncand);  // every lane walks the same tree
  float best = 3.402823466e+38f;   // per-lane running best
  uint32_t bestKey = 0xffffffffu;  // tree position of the lane's best candidate
  uint32_t bestIp = kInvalidPoly;
  float bp[3] = {0, 0, 0};
  int ncands = 0;  // candidates waiting in the batch (uniform)
  auto flush = [&]() {
    if (lane < ncands) {
      const uint32_t ip = L.cand_poly[lane];
      float cp[3];
      const float d = snap_candidate(nav, s, nav.polys[s.poly_base + ip], px, py, pz, cp);
      const uint32_t key = L.cand_node[lane];
      if (d < best || (d == best && d < 3.402823466e+38f && key < bestKey)) {
        best = d; bestKey = key; bestIp = ip; bp[0] = cp[0]; bp[1] = cp[1]; bp[2] = cp[2];
      }
    }
    *ncand += (uint32_t)ncands;
    ncands = 0;
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };
  // roots: the tree proper and whatever the builder left behind it in the array
  int nf = 0, cur = 0;
  {
    uint32_t k = 0;
    while (k < s.bv_count && nf < kSnapFrontier) {
      if (lane == 0) L.frontier[0][nf] = (uint16_t)k;
      nf++;
      const BVNodeDev nd = nav.bv[s.bv_base + k];
      k += nd.b == kBVLeaf ? 1u : (uint32_t)nd.a;
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  bool overflow = false;
  while (nf > 0 && !overflow) {
    int nnext = 0;
    for (int basei = 0; basei < nf; basei += 64) {
      const int fi = basei + lane;
      bool isCand = false, isInner = false;
      uint32_t node = 0;
      BVNodeDev nd{};
      if (fi < nf) {
        node = L.frontier[cur][fi];
        nd = nav.bv[s.bv_base + node];
        bool overlap = true;
#pragma unroll
        for (int k = 0; k < 3; ++k)
          if (box.bmin[k] > nd.bmax[k] || box.bmax[k] < nd.bmin[k]) overlap = false;
        if (overlap) {
          if (nd.b == kBVLeaf) isCand = (nav.polys[s.poly_base + nd.a].flags & 1) != 0;
          else isInner = true;
        }
      }
      // children of overlapping inner nodes go to the next frontier
      const unsigned long long mi = __ballot(isInner);
      const int ni = __popcll(mi);
      if (nnext + 2 * ni > kSnapFrontier) { overflow = true; break; }
      if (isInner) {
        const int pos = nnext + 2 * __popcll(mi & ((1ull << lane) - 1ull));
        L.frontier[cur ^ 1][pos] = (uint16_t)(node + 1);
        L.frontier[cur ^ 1][pos + 1] = nd.b;
      }
      nnext += 2 * ni;
      // overlapping walkable leaves join the candidate batch; a full batch is evaluated
      unsigned long long mc = __ballot(isCand);
      while (mc) {
        const int room = 64 - ncands;
        const int take = min(room, (int)__popcll(mc));
        const int rank = __popcll(mc & ((1ull << lane) - 1ull));
        if (isCand && rank < take) {
          L.cand_node[ncands + rank] = (uint16_t)node;
          L.cand_poly[ncands + rank] = nd.a;
          isCand = false;
        }
        ncands += take;
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (ncands == 64) flush();
        mc = __ballot(isCand);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
    cur ^= 1;
    nf = nnext;
  }
  if (overflow) return snap_point(nav, s, px, py, pz, ncand);
  if (ncands) flush();
  // wave-wide minimum of (distance, tree position)
  for (int o = 32; o > 0; o >>= 1) {
    const float od = __shfl_xor(best, o);
    const uint32_t ok = (uint32_t)__shfl_xor((int)bestKey, o);
    const uint32_t oi = (uint32_t)__shfl_xor((int)bestIp, o);
    const float o0 = __shfl_xor(bp[0], o), o1 = __shfl_xor(bp[1], o), o2 = __shfl_xor(bp[2], o);
    const bool mineValid = bestIp != kInvalidPoly, otherValid = oi != kInvalidPoly;
    const bool takeOther = otherValid && (!mineValid || od < best || (od == best && ok < bestKey));
    if (takeOther) { best = od; bestKey = ok; bestIp = oi; bp[0] = o0; bp[1] = o1; bp[2] = o2; }
  }
  if (bestIp == kInvalidPoly || isnan(bp[0])) return out;
  out.x = bp[0]; out.y = bp[1]; out.z = bp[2];
  out.ref = s.ref_base | bestIp;
  return out;
}

// A polygon record in registers, for the move of one agent per lane: its first 112 bytes arrive
// with seven 16-byte loads that go out together, where the loops over a record in memory pay a
// load and a wait for every field as they come to it (a forward move is one chain of dependent
// loads: state, scene, polygon, neighbour polygon, height mesh).  Every index into the words is
// a compile-time constant: loops over vertices are unrolled in the source (static_for), and a
// vertex or neighbour code with a run-time index is picked by a chain of selects whose operands
// the optimiser cannot trace back to the array (PolyRegs::reg), because either an index that
// is still a loop variable or a select between two loads of the array makes it an array in
// scratch memory again.  Same float operations in the same order as the versions on records
// in memory above.
// (lambdas handed to static_for are marked BPSX_INLINE_LAMBDA: inlined together with the functions
// around them, before the optimiser first looks at the record)
#define BPSX_INLINE_LAMBDA __attribute__((always_inline))
template <int I> struct Idx { static constexpr int value = I; };
template <int B, int E, class F> BPSX_DEV void static_for(F&& f) {
  if constexpr (B < E) {
    f(Idx<B>{});
    static_for<B + 1, E>(f);
  }
}
struct PolyRegs {
  uint32_t w[28];
  BPSX_DEV void load(const PolyRec* p) {
    const uint4* s = reinterpret_cast<const uint4*>(p);
    static_for<0, 7>([&](auto K) BPSX_INLINE_LAMBDA {
      constexpr int k = decltype(K)::value;
      const uint4 q = s[k];
      w[4 * k] = q.x; w[4 * k + 1] = q.y; w[4 * k + 2] = q.z; w[4 * k + 3] = q.w;
    });
  }
  static_assert(offsetof(PolyRec, nei) == 72 && offsetof(PolyRec, walk) == 84 && offsetof(PolyRec, flags) == 96 &&
                offsetof(PolyRec, nv) == 98 && offsetof(PolyRec, type) == 99 && offsetof(PolyRec, tri_base) == 100 &&
                offsetof(PolyRec, dvert_base) == 104 && offsetof(PolyRec, tri_count) == 108, "PolyRegs follows PolyRec's layout");
  template <int I> BPSX_DEV float x() const { return __uint_as_float(w[3 * I]); }
  template <int I> BPSX_DEV float y() const { return __uint_as_float(w[3 * I + 1]); }
  template <int I> BPSX_DEV float z() const { return __uint_as_float(w[3 * I + 2]); }
  template <int J> BPSX_DEV uint32_t nei() const { return (w[18 + (J >> 1)] >> (16 * (J & 1))) & 0xffffu; }
  template <int J> BPSX_DEV uint32_t walk() const { return (w[21 + (J >> 1)] >> (16 * (J & 1))) & 0xffffu; }
  BPSX_DEV int nv() const { return (int)((w[24] >> 16) & 0xffu); }
  BPSX_DEV uint32_t type() const { return w[24] >> 24; }
  BPSX_DEV uint32_t tri_base() const { return w[25]; }
  BPSX_DEV uint32_t dvert_base() const { return w[26]; }
  BPSX_DEV int tri_count() const { return (int)(w[27] & 0xffu); }
  // vertex k, k known at run time only.  The words pass through an empty asm first: selects
  // between loads of the array would be folded into one load at a selected address, and the
  // record would have to live in (scratch) memory for it.
  static BPSX_DEV uint32_t reg(uint32_t v) { asm("" : "+v"(v)); return v; }
  BPSX_DEV uint32_t word(int k, int stride, int base) const {   // w[base + stride * k], k in 0..5
    const uint32_t a0 = reg(w[base]), a1 = reg(w[base + stride]), a2 = reg(w[base + 2 * stride]), a3 = reg(w[base + 3 * stride]),
                   a4 = reg(w[base + 4 * stride]), a5 = reg(w[base + 5 * stride]);
    return k == 5 ? a5 : k == 4 ? a4 : k == 3 ? a3 : k == 2 ? a2 : k == 1 ? a1 : a0;
  }
  BPSX_DEV void vertex(int k, float* o) const {
    o[0] = __uint_as_float(word(k, 3, 0));
    o[1] = __uint_as_float(word(k, 3, 1));
    o[2] = __uint_as_float(word(k, 3, 2));
  }
  BPSX_DEV void codes(int k, uint32_t* nei_k, uint32_t* walk_k) const {
    const uint32_t n = word(k >> 1, 1, 18), wk = word(k >> 1, 1, 21);   // two 16-bit codes per word; k >> 1 in 0..2
    *nei_k = (n >> (16 * (k & 1))) & 0xffffu;
    *walk_k = (wk >> (16 * (k & 1))) & 0xffffu;
  }
};

BPSX_DEV bool point_in_poly(float px, float pz, const PolyRegs& P) {
  bool c = false;
  const int nv = P.nv();
  float vj[3];
  P.vertex(nv - 1, vj);
  float jx = vj[0], jz = vj[2];
  static_for<0, kNvp>([&](auto I) BPSX_INLINE_LAMBDA {
    constexpr int i = decltype(I)::value;
    const float ix = P.x<i>(), iz = P.z<i>();
    const bool crosses = ((iz > pz) != (jz > pz)) && (px < (jx - ix) * (pz - iz) / (jz - iz) + ix);
    c ^= (i < nv) && crosses;
    jx = ix; jz = iz;
  });
  return c;
}

// dtNavMesh::getPolyHeight on a record in registers (`mem`: the same record in memory, for the
// rare fall-back to the detail edges).  The index words of the first four detail triangles go
// out together.
BPSX_DEV bool poly_height(const NavData& nav, const PolyRegs& P, const PolyRec& mem, float px, float py, float pz, float& h) {
  if (P.type() != 0) return false;
  if (!point_in_poly(px, pz, P)) return false;
  const int tc = P.tri_count(), nv = P.nv();
  const uint32_t* tris = reinterpret_cast<const uint32_t*>(nav.dtris) + P.tri_base();   // four bytes per triangle
  const uint32_t t0 = 0 < tc ? tris[0] : 0u, t1 = 1 < tc ? tris[1] : 0u, t2 = 2 < tc ? tris[2] : 0u, t3 = 3 < tc ? tris[3] : 0u;
  auto corner = [&](uint32_t k, float* o) BPSX_INLINE_LAMBDA {
    if ((int)k < nv) P.vertex((int)k, o);
    else {
      const float* d = &nav.dverts[(size_t)(P.dvert_base() + (k - (uint32_t)nv)) * 3];
      o[0] = d[0]; o[1] = d[1]; o[2] = d[2];
    }
  };
  auto inside = [&](uint32_t t) BPSX_INLINE_LAMBDA {
    float a[3], b[3], c[3];
    corner(t & 0xffu, a); corner((t >> 8) & 0xffu, b); corner((t >> 16) & 0xffu, c);
    return height_on_triangle(px, pz, a, b, c, h);
  };
  if (0 < tc && inside(t0)) return true;
  if (1 < tc && inside(t1)) return true;
  if (2 < tc && inside(t2)) return true;
  if (3 < tc && inside(t3)) return true;
  for (int j = 4; j < tc; ++j)
    if (inside(tris[j])) return true;
  float c[3];
  closest_on_detail_edges<false>(nav, mem, px, py, pz, c);
  h = c[1];
  return true;
}

// The tiny node pool and the queue of moveAlongSurface, one column per lane of a wavefront, in
// LDS: they are indexed at run time, which in private memory means a trip to scratch (HBM
// behind the vector caches) per access.  A node enters the queue at most once, so the queue
// needs no more entries than there are nodes and is never shifted: `head` moves instead.
struct MoveLds {
  uint16_t node_id[kTinyNodes][64];
  uint8_t queue[kTinyNodes][64];
};

// tryStep with sliding, one lane per agent.
BPSX_DEV NavPt try_step(const NavData& nav, const SceneDev& s, const NavPt& start, float ex, float ey, float ez,
                        uint32_t* npolys, MoveLds& M) {
  const uint32_t startIp = decode_ref(s, start.ref);
  if (startIp == kInvalidPoly || !finite3(start.x, start.y, start.z) || !finite3(ex, ey, ez)) return start;
  const int lane = (int)(threadIdx.x & 63);
  uint64_t closed = 1ull;
  int nnodes = 1;
  int qhead = 0, qtail = 1;   // the reference's stack holds entries [qhead, qtail)
  M.node_id[0][lane] = (uint16_t)startIp;
  M.queue[0][lane] = 0;
  float bx = start.x, by = start.y, bz = start.z;
  float bestDist = 3.402823466e+38f;
  int bestNode = -1;
  const float sx = start.x + (ex - start.x) * 0.5f, sz = start.z + (ez - start.z) * 0.5f;
  const float ddx = ex - start.x, ddy = ey - start.y, ddz = ez - start.z;
  const float sr = sqrtf(ddx * ddx + ddy * ddy + ddz * ddz) / 2.0f + 0.001f;
  const float searchRadSqr = sr * sr;
  PolyRegs P;
  uint32_t loaded = kInvalidPoly;   // the polygon P holds
  while (qhead < qtail) {
    const int cur = M.queue[qhead++][lane];
    loaded = M.node_id[cur][lane];
    P.load(&nav.polys[s.poly_base + loaded]);
    (*npolys)++;
    if (point_in_poly(ex, ez, P)) {
      bestNode = cur;
      bx = ex; by = ey; bz = ez;
      break;
    }
    const int nv = P.nv();
    // edge j -> i with j the vertex before i: (nv - 1, 0), (0, 1), ...
    float vj[3];
    uint32_t neij, walkj;
    P.vertex(nv - 1, vj);
    P.codes(nv - 1, &neij, &walkj);
    static_for<0, kNvp>([&](auto I) BPSX_INLINE_LAMBDA {
      constexpr int i = decltype(I)::value;
      const float vi[3] = {P.x<i>(), P.y<i>(), P.z<i>()};
      if (i < nv) {
        // single-tile meshes carry no tile-border links, so a border edge is a wall
        const uint32_t nb = (neij & 0x8000u) ? 0u : walkj;
        if (!nb) {
          float t;
          const float d = dist_pt_seg_sqr2d(ex, ez, vj, vi, t);
          if (d < bestDist) {
            bx = vj[0] + (vi[0] - vj[0]) * t;
            by = vj[1] + (vi[1] - vj[1]) * t;
            bz = vj[2] + (vi[2] - vj[2]) * t;
            bestDist = d;
            bestNode = cur;
          }
        } else {
          const uint16_t ip = (uint16_t)(nb - 1);
          int nn = -1;
          for (int k = 0; k < nnodes; ++k)
            if (M.node_id[k][lane] == ip) { nn = k; break; }
          bool fits = true;
          if (nn < 0) {
            if (nnodes >= kTinyNodes) fits = false;
            else {
              nn = nnodes++;
              M.node_id[nn][lane] = ip;
            }
          }
          if (fits && !((closed >> nn) & 1ull)) {
            float t;
            const float d = dist_pt_seg_sqr2d(sx, sz, vj, vi, t);
            if (!(d > searchRadSqr) && qtail - qhead < kMoveQueue) {
              closed |= 1ull << nn;
              M.queue[qtail++][lane] = (uint8_t)nn;
            }
          }
        }
      }
      vj[0] = vi[0]; vj[1] = vi[1]; vj[2] = vi[2];
      neij = P.nei<i>(); walkj = P.walk<i>();
    });
  }
  if (bestNode < 0) return start;
  const uint32_t bestIp = M.node_id[bestNode][lane];
  NavPt out{bx, by, bz, s.ref_base | bestIp};
  if (isfinite(bx) && isfinite(bz)) {
    const PolyRec& mem = nav.polys[s.poly_base + bestIp];
    if (bestIp != loaded) P.load(&mem);
    float h;
    if (poly_height(nav, P, mem, bx, by, bz, h)) out.y = h;
  }
  return out;
}

// dtRandomPointInConvexPoly on a polygon record.
BPSX_DEV void random_point_in_poly(const PolyRec& r, float sv, float tv, float* out) {
  float areas[kNvp];
  float areasum = 0.0f;
  const int n = r.nv;
  for (int i = 2; i < n; i++) {
    const float abx = r.v[i - 1][0] - r.v[0][0], abz = r.v[i - 1][2] - r.v[0][2];
    const float acx = r.v[i][0] - r.v[0][0], acz = r.v[i][2] - r.v[0][2];
    areas[i] = acx * abz - abx * acz;
    areasum += areas[i] > 0.001f ? areas[i] : 0.001f;
  }
  const float thr = sv * areasum;
  float acc = 0.0f, u = 1.0f;
  int tri = n - 1;
  for (int i = 2; i < n; i++) {
    const float dacc = areas[i];
    if (thr >= acc && thr < (acc + dacc)) { u = (thr - acc) / dacc; tri = i; break; }
    acc += dacc;
  }
  const float v = sqrtf(tv);
  const float a = 1 - v, b = (1 - u) * v, c = u * v;
  const float* pa = r.v[0];
  const float* pb = r.v[tri - 1];
  const float* pc = r.v[tri];
  out[0] = a * pa[0] + b * pb[0] + c * pc[0];
  out[1] = a * pa[1] + b * pb[1] + c * pc[1];
  out[2] = a * pa[2] + b * pb[2] + c * pc[2];
}

// Area-weighted polygon pick + point: first polygon whose inclusive area prefix sum exceeds
// u0 * total, then a point inside it, y from the height mesh.
BPSX_DEV bool sample_point(const NavData& nav, const SceneDev& s, float u0, float sv, float tv, float* out,
                           uint32_t* out_ip) {
  if (!(s.area_total > 0.0f)) return false;
  const float target = u0 * s.area_total;
  uint32_t lo = 0, hi = s.poly_count - 1;
  while (lo < hi) {
    const uint32_t mid = (lo + hi) / 2;
    if (nav.polys[s.poly_base + mid].area_cum > target) hi = mid;
    else lo = mid + 1;
  }
  const PolyRec& r = nav.polys[s.poly_base + lo];
  random_point_in_poly(r, sv, tv, out);
  float h;
  if (isfinite(out[0]) && isfinite(out[2]) && poly_height(nav, r, out[0], out[1], out[2], h)) out[1] = h;
  *out_ip = lo;
  return true;
}

}  // namespace bpsx
