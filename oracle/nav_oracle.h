// TEST INFRASTRUCTURE — CPU restatement of the reference's navmesh query path.
//
// This is the checker that the HIP kernels are compared against, never the product:
// only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it.
//
// It restates, in independent code, the algorithms of
//   PathFinder.cpp  (habitat_sim_geodesic/csrc): loadNavMesh :330-408, removeZeroAreaPolys
//                   :276-328, IslandSystem :53-170, snapPoint :573-584 / projectToPoly :24-44,
//                   tryStep :543-571, findPathInternal :485-526, pathLength :473-482
//   DetourNavMesh.cpp: init :224-265, addTile :908-1048 (single tile), connectIntLinks
//                   :524-559, getPolyHeight :677-726, closestPointOnPoly :728-758,
//                   closestPointOnDetailEdges :619-675
//   DetourNavMeshQuery.cpp: findNearestPoly :685-709 (+ :642-676, :711-826, :895-932),
//                   moveAlongSurface :2016-2255, findPath :945-1178, findStraightPath
//                   :1765-1994 (+ appendVertex :1661-1696, closestPointOnPolyBoundary
//                   :538-586, getPortalPoints :2279-2349), findRandomPoint sampling :220-313
//   DetourCommon.{h,cpp}, DetourNode.{h,cpp}: geometry primitives, node pool, heap.
//
// Parity status: every function here is pinned bit-exactly against the compiled reference
// (oracle/_ref) by tests/test_oracle_vs_ref.py in the development container, and against the
// golden traces that build wrote into tests/golden/ everywhere else.
// Multi-tile navmeshes (tile-border links) are not restated: load() rejects them.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace orc {

struct NavPoint {
  float xyz[3];
  uint32_t ref;  // Detour-encoded polygon ref, 0 = none
};

// Work counters for the algorithmic-bytes model of the step path.
struct Counters {
  uint64_t move_calls = 0;      // moveAlongSurface invocations
  uint64_t move_polys = 0;      // polygons dequeued by the moves
  uint64_t move_verts = 0;      // vertices of those polygons
  uint64_t height_tris = 0;     // detail triangles of polygons whose height was taken
  uint64_t path_calls = 0;      // geodesic queries that reached A*
  uint64_t astar_pops = 0;      // nodes expanded
  uint64_t astar_links = 0;     // links scanned
  uint64_t corridor_polys = 0;  // sum of corridor lengths handed to the funnel
  uint64_t snap_calls = 0;
  uint64_t snap_bv_nodes = 0;   // BV nodes tested
  uint64_t snap_cands = 0;      // candidate polygons
  uint64_t snap_cand_verts = 0;
  uint64_t snap_cand_tris = 0;
  void add(const Counters& o);
};

class Mesh;
// Parses MSET bytes; returns nullptr and sets *err on failure. The mesh is immutable
// afterwards and may be shared by any number of Query objects.
Mesh* mesh_load(const uint8_t* bytes, size_t n, std::string* err);
void mesh_free(Mesh* m);
int mesh_poly_count(const Mesh* m);
uint32_t mesh_poly_ref(const Mesh* m, int poly_index);
// flags after zero-area disabling, island id per polygon
uint16_t mesh_poly_flags(const Mesh* m, int poly_index);
int mesh_poly_island(const Mesh* m, int poly_index);

// dtRandomPointInConvexPoly (DetourCommon.cpp:332-369). areas: scratch of npts floats.
void random_point_in_convex_poly(const float* pts, int npts, float* areas, float s, float t, float* out);

// Mutable query context (node pools); one per thread.
class Query {
 public:
  explicit Query(const Mesh* mesh);
  ~Query();
  NavPoint snapPoint(const float* pt);
  NavPoint tryStep(const NavPoint& start, const float* end);
  float geodesic(const NavPoint& start, const NavPoint& end);
  // The distance-field formulation of the same query (NOT the reference's algorithm; only for
  // measuring how far it is from geodesic()): parent chain of a goal-rooted Dijkstra search as
  // the corridor, then the same string pulling.
  float geodesicViaField(const NavPoint& start, const NavPoint& end);
  // Corridor of the last geodesic() that reached the funnel (polygon refs).
  const std::vector<uint32_t>& lastCorridor() const { return corridor_; }
  // Area-weighted pick: polygon by u0 over the float prefix sum of fan areas, then
  // random_point_in_convex_poly(s, t), y from the height mesh. Returns false if the mesh
  // has no walkable area.
  bool samplePoint(float u0, float s, float t, float* out_xyz, uint32_t* out_ref);
  Counters counters;
  // Check of the rules by which the GPU kernel expands several open nodes per pass (TEST
  // INFRASTRUCTURE like the rest of this file).  With rows > 0, geodesic() predicts before a
  // pop, from the open list sorted by total and the state as it is, which nodes the next pops
  // will be and what their expansions will write, by the kernel's rules: entry j stands while its
  // total is below entry j + 1's, no earlier entry's update reaches its total or touches a
  // polygon it reads, and it is not the goal; two entries that share the smallest total stand
  // together, in either order, when neither touches what the other reads.  The search itself is
  // the reference's, unchanged; every prediction is compared with what it then does.
  struct PassCheck {
    int rows = 0;
    uint64_t passes = 0, nodes = 0;        // predictions made, pops they covered
    uint64_t wrongNode = 0, wrongUpdate = 0;   // pops of another node / expansions that wrote something else
    uint64_t pairs = 0, ties = 0;          // tied pairs predicted as a pair / ties left to the heap
  } passCheck;

 private:
  struct Impl;
  const Mesh* mesh_;
  Impl* impl_;
  std::vector<uint32_t> corridor_;
  float corridorLength(const NavPoint& start, const NavPoint& end);
  struct Field {
    uint32_t rootRef = 0;
    float root[3] = {0, 0, 0};
    std::vector<int> parent;
    std::vector<float> pos, cost;
  } field_;
};

}  // namespace orc
