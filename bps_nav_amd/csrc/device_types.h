// Layout of the navmesh and agent data in HBM, shared by the host uploader and the kernels.
//
// Polygons are stored as one 128-byte record each (one L2 cache line on gfx950), so a walk
// that hops from polygon to polygon costs exactly one line per hop: vertices, neighbours,
// filter result and the handle of the height mesh travel together.  Everything an agent
// gathers per step is indexed by (scene polygon base + polygon index).
#pragma once
#include <cstdint>

namespace bpsx {

constexpr int kNvp = 6;
constexpr uint32_t kInvalidPoly = 0xffffffffu;

// Detour buffer limits that are part of the reference's observable behaviour.
constexpr int kMaxNodes = 2048;     // dtNavMeshQuery::init(nav, 2048), PathFinder.cpp:247
constexpr int kMaxPath = 256;       // MAX_POLYS, PathFinder.cpp:499, 546
constexpr int kTinyNodes = 64;      // m_tinyNodePool, DetourNavMeshQuery.cpp:191
constexpr int kMoveQueue = 48;      // MAX_STACK, DetourNavMeshQuery.cpp:2039

struct alignas(128) PolyRec {
  float v[kNvp][3];        // vertex positions, polygon order
  uint16_t nei[kNvp];      // raw Detour neis: 0 wall, idx+1 internal, 0x8000|dir tile border
  uint16_t walk[kNvp];     // idx+1 of the neighbour across edge j if it passes the query
                           // filter (PathFinder.cpp:239-243), else 0
  uint16_t flags;          // polygon flags after zero-area disabling (PathFinder.cpp:307-328)
  uint8_t nv;              // vertex count
  uint8_t type;            // 0 ground, 1 off-mesh connection
  uint32_t tri_base;       // first detail triangle, index into the global triangle array
  uint32_t dvert_base;     // first extra detail vertex, index into the global array
  uint8_t tri_count;
  uint8_t dvert_count;
  uint16_t pad0;
  uint32_t island;         // connected component id (IslandSystem, PathFinder.cpp:53-170)
  float area_cum;          // inclusive prefix sum of walkable fan areas (sampling)
  uint32_t pad1[2];
};
static_assert(sizeof(PolyRec) == 128, "PolyRec must be one cache line");

// What A* needs of one polygon edge: where a path crossing it is taken to pass (the midpoint
// of the portal, getEdgeMidPoint in DetourNavMeshQuery.cpp:2352-2381, computed once at upload
// with the same float operations) and which polygon lies behind it.  Six of them per polygon,
// so lane j of a wavefront fetches edge j of the expanded polygon with one 16-byte load.
struct AEdge {
  float mid[3];
  uint32_t nb;   // polygon index behind the edge if the search may enter it (internal link to
                 // a polygon that passes the query filter), else kNoNb
};
static_assert(sizeof(AEdge) == 16, "AEdge");
constexpr int kEdgeStride = 8;   // records per polygon in HBM: six edges and two unused, one 128-byte line
constexpr uint32_t kNoNb = 0xffffu;

// dtBVNode repacked at upload: same quantised bounds; a leaf carries its polygon index, an
// internal node carries Detour's escape offset (for the in-order walk) and the index of its
// right child (its left child is the next node), so a wavefront can descend level by level.
struct BVNodeDev {
  uint16_t bmin[3], bmax[3];
  uint16_t a;   // leaf: polygon index; internal: escape offset
  uint16_t b;   // leaf: 0xffff; internal: index of the right child
};
static_assert(sizeof(BVNodeDev) == 16, "BV node");
constexpr uint16_t kBVLeaf = 0xffff;

struct SceneDev {
  uint32_t poly_base, poly_count;
  uint32_t bv_base, bv_count;
  uint32_t ep_base, ep_count;       // rows of 10 floats in the episode array
  uint32_t ref_base;                // salt and tile bits of every polygon ref of the scene
  uint32_t poly_mask;               // (1 << polyBits) - 1
  float orig[3], tile_w, tile_h;    // dtNavMeshParams
  int32_t tx, ty;                   // tile grid location
  float bmin[3], bmax[3];           // tile bounds
  float qfac;                       // bvQuantFactor
  float climb;                      // walkableClimb
  float area_total;
  uint32_t bv_tree_ok;              // 1: child links verified, level-by-level descent allowed
  uint32_t pad[2];
};

// ---- per-agent state, structure of arrays over all agents of the simulator
struct AgentArrays {
  float* pos;         // [N][3]
  float* rot;         // [N][4] x,y,z,w
  float* goal;        // [N][3]
  float* nav_xyz;     // [N][3] navmeshPosition_.xyz
  uint32_t* nav_ref;  // [N]    navmeshPosition_.polyId
  float* goal_xyz;    // [N][3] navmeshGoal_.xyz
  uint32_t* goal_ref; // [N]
  float* prev_pos;    // [N][3]
  float* info_prev;   // [N] InfoFunctor::prev_distance_to_goal_
  float* cum;         // [N]
  float* init;        // [N]
  float* rew_prev;    // [N] RewardFunctor::prev_distance_to_goal_
  uint32_t* step;     // [N]
  uint32_t* scene;    // [N]
  uint32_t* episode;  // [N]
  uint32_t* nresets;  // [N]
  uint32_t* flags;    // [N] transient per-step bits, see kAgent*
  uint32_t* dist_ok;  // [N] 1 when info_prev is the goal->agent distance of the current navmesh point
  uint32_t* last_cost;// [N] nodes expanded by the agent's most recent path search (scheduling hint)
  float* geo;         // [2N] geodesic results: [i] step query of agent i, [N + i] its reset query
  // Exploration task only
  float* exp_init;    // [N][3] position at reset
  float* exp_inv;     // [N][4] inverse of the rotation at reset
  int32_t* exp_cells; // [N][cell_cap][3] cells entered this episode
  uint32_t* exp_count;// [N]
  uint32_t cell_cap;  // one cell per step at most: max_steps
  // outputs
  float* rewards;     // [N]
  uint8_t* masks;     // [N]
  float* infos;       // [N][3]
  float* polars;      // [N][2]
};
constexpr uint32_t kAgentDone = 1u, kAgentMoved = 2u, kAgentReuse = 4u, kAgentSkip = 8u, kAgentResetOnly = 16u;

struct NavData {
  const PolyRec* polys;
  const AEdge* aedges;     // [polygon][kEdgeStride]
  const BVNodeDev* bv;
  const uint8_t* dtris;    // [.][4]
  const float* dverts;     // [.][3]
  const SceneDev* scenes;
  const float* episodes;   // [.][10]
};

// A* node of the per-slot pool (dtNode, DetourNode.h:36-45) as kept in HBM: 32 bytes.
struct alignas(16) ANode {
  float pos[3];
  float cost;
  float total;
  uint32_t parent;  // 1-based index of the node this one was reached from, 0 for the start node
  uint32_t link;    // polygon index within the scene (bits 0-14) | flags (bits 15-16: 1 open, 2 closed) | next node of the hash chain << 20
  uint32_t pad;
};
static_assert(sizeof(ANode) == 32, "ANode");

struct HeapEntry {
  float total;
  uint32_t node;
};

// HBM slot of one A* wavefront: the node pool (LDS caches its hot part) and the open-list
// entries beyond what LDS holds.
// Record of the open-list operations of a search that keeps its open list sorted (see
// geodesic_device.h): per pass one header (key = number of entries popped | number of records
// that follow << 8, word = kOpHeader) followed by the pass's pushes and modifies in row and
// edge order (key = total as bits, word = packed node | row of the pass << 26 | 1 << 29 if the
// node was open).  A header with kOpUnordered says that the pass's first two rows had the same
// total: the reference expanded them in the order its heap had them in, which the replay finds
// out; the header's low 26 bits then name row 0's node.
struct OpRec {
  uint32_t key;
  uint32_t word;
};
constexpr uint32_t kOpHeader = 0x80000000u, kOpUnordered = 0x40000000u;
constexpr int kOpLogCap = 8192;

struct alignas(128) GeoSlot {
  ANode nodes[kMaxNodes];
  HeapEntry heap_spill[kMaxNodes];
  OpRec oplog[kOpLogCap];
  uint16_t parents[kMaxNodes];   // the nodes' parent indices once more, side by side: what the final walk up the path reads
};

struct GeoQuery {
  float a[3];
  uint32_t a_ref;
  float b[3];
  uint32_t b_ref;
  uint32_t scene;
  uint32_t out;   // index into the result array
  uint32_t cost_slot;  // agent whose cost estimate this query refreshes, or kNoCostSlot
  uint32_t pad;
};
constexpr uint32_t kNoCostSlot = 0xffffffffu;

// Path searches differ in length by two orders of magnitude and each is sequential, so a step
// ends when its longest search ends.  Queries are therefore queued in classes of expected
// cost (the nodes the agent's previous searches expanded) and served from the longest class
// down, which approximates longest-first scheduling; the longer classes also run at a higher
// issue priority of their wavefront.
// The classes are narrow because tickets within a class are served in the order they were
// queued: the last searches to begin decide when a launch ends, and a class as wide as those
// searches are long lets one of its longest begin last.
#ifndef BPSX_GEO_CLASSES
#define BPSX_GEO_CLASSES 32
#endif
constexpr int kGeoClasses = BPSX_GEO_CLASSES;
constexpr uint32_t kGeoClassWidth = 2048 / BPSX_GEO_CLASSES;   // expanded nodes per class: the last class holds the shortest searches
constexpr __host__ __device__ uint32_t geo_class(uint32_t last_cost) {
  return last_cost / kGeoClassWidth >= (uint32_t)kGeoClasses ? 0u
                                                             : (uint32_t)kGeoClasses - 1u - last_cost / kGeoClassWidth;
}
// A search without history (one in ten) is queued as if it took 1000 nodes: about twice the mean,
// because one that turns out long and began late is what a launch then waits for, and one that
// turns out short and began early costs nothing.
constexpr uint32_t kGeoClassUnknown = geo_class(1000);
// AgentArrays::last_cost before the episode's first goal -> agent search.  The distance taken at
// reset is searched the other way round and the previous episode's searches had another goal:
// neither says how long the first search will be, and it is often among the longest.
constexpr uint32_t kCostUnknown = 0xffffffffu;

enum Counter {
  kCntSteps = 0, kCntForward, kCntGeoQueries, kCntAstarPops, kCntCorridor, kCntResets, kCntMovePolys, kCntSnapCands,
  kCntLinkSpills = 16, kCntHeapSpills = 17, kCntLongPath = 18, kCntExactRuns = 19, kCntTieReplays = 20, kCntPairTies = 21   // 8..15: phase cycles of the diagnostic build
};

}  // namespace bpsx
