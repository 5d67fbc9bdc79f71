// Geodesic distance on the GPU: Detour's A* over the polygon graph followed by the funnel
// (string pulling) and the summed segment length, with the exact buffer limits and failure
// conventions of the reference, so that the value equals PathFinder::findPath's.
//
// Execution model: one wavefront (64 lanes) owns one query at a time and pulls the next from
// a shared queue when done.  The search touches almost only nodes it created recently (the
// frontier of A* is narrow), so LDS holds what is hot and small and HBM holds the rest:
//   - the open list, a binary heap, in registers while it has fewer than 128 entries (entry q
//     in lane q mod 64); a longer one (rare) keeps its top kHeapLds entries in LDS,
//   - the hash heads of the node pool,
//   - for the first kLinksLds nodes one word with the polygon id, the open/closed flags and the
//     hash chain link (the parent index is read once per expansion and lives in HBM only),
//   - the position, cost and total of the kWindow most recently created nodes (slot = index
//     modulo kWindow) and their parent index; every write of those also goes to the
//     wavefront's slot in HBM, so an older node is simply read from there.
// Heap entries beyond kHeapLds and links beyond kLinksLds spill to the same slot.  A query
// runs the instantiation of the loop without spill code until one more expansion could
// outgrow the links in LDS or the register heap, then carries on in a spilling instantiation.
// Per expanded node the regular HBM traffic is the polygon's six 16-byte edge records (lane j
// of the wavefront handles edge j: node lookup, cost, heuristic) plus the write-through of
// updated nodes; heap updates are applied in edge order, which is what makes the result
// identical to the sequential algorithm, ties included.  A wavefront spends its time in one
// chain of dependent steps, so the code is written for few of them: heap pops and pushes are
// done by all lanes at once, what is the same for all lanes lives in scalar registers, and
// LDS and HBM accesses stay separate instructions.
//
// Reference semantics followed: DetourNavMeshQuery.cpp:945-1178 (findPath, getPathToNode),
// :1661-1696, 1765-1994 (appendVertex, findStraightPath), :2279-2381 (getPortalPoints,
// getEdgeMidPoint); DetourNode.cpp:50-200 (node pool, heap order); PathFinder.cpp:473-541.
//
// The sizes of the LDS structures are build parameters (BPSX_LINKS_LDS, BPSX_HEAP_LDS,
// BPSX_WINDOW, BPSX_HASH), and everything that depends on them lives in namespace
// bpsx::BPSX_GEO_NS (default geo): the file can be included again with other values and
// another namespace name to get a second instantiation of the same search.
#include "nav_device.h"

#ifndef BPSX_GEODESIC_COMMON_H
#define BPSX_GEODESIC_COMMON_H
#ifndef BPSX_BAG
#define BPSX_BAG 1   // 1: searches start with the open list as an unordered set (see OpenBag)
#endif
namespace bpsx {

#ifdef BPSX_ASM_MARKS
#define PHASE_MARK(k) asm volatile("; PHASE_MARK " #k)
#elif defined(BPSX_PHASE_TIMING)
#define PHASE_MARK(k) do { const unsigned long long now_ = __builtin_readcyclecounter(); phase_acc[k] += now_ - phase_t0; phase_t0 = now_; } while (0)
#else
#define PHASE_MARK(k) do { } while (0)
#endif

BPSX_DEV void wave_sync() {
  // All lanes belong to one wavefront: LDS and memory operations issue in program order, so
  // only the compiler has to be kept from reordering across this point.
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();
}
// Keeps the compiler from folding an LDS access and an HBM access of two branches into one
// generic-address access (which would wait on both memory counters and on pending stores).
#define BPSX_KEEP_APART() asm volatile("")
// s_setprio takes an immediate
BPSX_DEV void set_wave_priority(int p) {
  if (p >= 3) __builtin_amdgcn_s_setprio(3);
  else if (p == 2) __builtin_amdgcn_s_setprio(2);
  else if (p == 1) __builtin_amdgcn_s_setprio(1);
  else __builtin_amdgcn_s_setprio(0);
}
BPSX_DEV int uniform_i(int v) { return __builtin_amdgcn_readfirstlane(v); }
BPSX_DEV float uniform_f(float v) { return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v))); }
BPSX_DEV float lane_f(float v, int lane) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane)); }
BPSX_DEV int lane_i(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }
BPSX_DEV uint32_t rlane(uint32_t v, int lane) { return (uint32_t)__builtin_amdgcn_readlane((int)v, lane); }
// old with lane `lane` replaced by v (v and lane uniform).  The lane select travels in M0:
// gfx9 encodings take at most one general scalar register per vector instruction.
BPSX_DEV uint32_t wlane(uint32_t old, uint32_t v, int lane) {
  const int sv = __builtin_amdgcn_readfirstlane((int)v), sl = __builtin_amdgcn_readfirstlane(lane);
  asm("s_mov_b32 m0, %2\n\tv_writelane_b32 %0, %1, m0" : "+v"(old) : "s"(sv), "s"(sl) : "m0");
  return old;
}

// lanes 8..15 of each row of 16 take src of the lane 8 below them, lanes 0..7 keep low
BPSX_DEV float lanes_up8(float low, float src) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(low), __float_as_int(src), 0x118 /* row_shr:8 */, 0xf, 0xf, false));
}
// lanes 0..7 of each row take v of the lane 8 above them
BPSX_DEV float lanes_down8(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x108 /* row_shl:8 */, 0xf, 0xf, false));
}
// Correctly rounded square root, the value sqrtf returns on the host: the hardware estimate is
// within one unit in the last place, and the residuals of its two neighbours say which of the
// three is the rounded root.  Same scheme as the compiler's own expansion of sqrtf, minus its
// rescaling of arguments below 2^-96 (needed there for the residuals not to underflow): the
// arguments here are squared distances, zero or far above that; a wavefront that meets one in
// between takes the library routine.
BPSX_DEV float sqrt_exact(float x) {
  const uint32_t xb = __float_as_uint(x);
  if (__ballot(xb - 1u < 0x0f800000u - 1u)) return sqrtf(x);   // 0 < x < 2^-96 in some lane: never in practice
  const float s = __builtin_amdgcn_sqrtf(x);
  const float down = __uint_as_float(__float_as_uint(s) - 1u), up = __uint_as_float(__float_as_uint(s) + 1u);
  const float rdown = fmaf(-down, s, x), rup = fmaf(-up, s, x);
  float r = rdown <= 0.0f ? down : s;
  r = rup > 0.0f ? up : r;
  return r;
}

// One word per node holds what the search loop reads of it besides the window: the parent
// index is needed once per expansion and for the final path, and lives in HBM only.
constexpr uint32_t kChainEnd = 0xfffu;
static_assert(kMaxNodes <= (int)kChainEnd, "node indices must stay below the chain end marker");
BPSX_DEV uint32_t link_id(uint32_t l) { return l & 0x7fffu; }
BPSX_DEV uint32_t link_flags(uint32_t l) { return (l >> 15) & 3u; }
BPSX_DEV uint32_t link_next(uint32_t l) { return l >> 20; }
BPSX_DEV uint32_t make_link(uint32_t id, uint32_t flags, uint32_t next) { return id | (flags << 15) | (next << 20); }
BPSX_DEV uint32_t with_flags(uint32_t l, uint32_t flags) { return (l & ~(3u << 15)) | (flags << 15); }

// The open list in registers.  Heap position q (1-based, root = 1; the reference's index + 1)
// lives in lane q & 63 of the first register pair (q < 64) or of the second (64 <= q < 128).
// Totals are kept as bit patterns and compared as unsigned integers: they are sums of
// distances, never negative and never NaN, and for such floats the integer order of the bits
// is the float order.  Same algorithm as dtNodeQueue (DetourNode.cpp:150-200).
constexpr int kRegHeap = 127;
static_assert(kMaxNodes <= 2048, "heap entries keep the node index in 11 bits");
struct RegHeap {
  uint32_t t0, t1;   // total bits
  uint32_t n0, n1;   // node index (bits 0-10) | the node's polygon index << 11, so that popping
                     // the root names the edge records to fetch without a detour through LDS
  int size;
  static constexpr uint32_t kEmpty = 0x7fffffffu;   // above +inf; every key stays below 2^31
  BPSX_DEV void init() { t0 = t1 = kEmpty; n0 = n1 = 0; size = 0; }
  static BPSX_DEV uint32_t xlane(int src_lane, uint32_t v) {   // v of another lane; all lanes must be active
    return (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane * 4, (int)v);
  }

  // dtNodeQueue::bubbleUp of entry (t, n) from position q, by all lanes at once.  The lanes on
  // the way from q to the root read their parent's entry; ancestors with a greater key move
  // one step down that way (they form a run from q upwards: keys never increase towards the
  // root) and the entry lands on top of the run.  Positions 64..127 have all their ancestors
  // in the first pair, so only q itself can be in the second.
  BPSX_DEV void bubble_up(int q, uint32_t t, uint32_t n, int lane) {
    const int up = (31 - __clz(q)) - (31 - __clz(lane));   // lane 0 (clz 32) is no heap position
    const bool on = lane >= 1 && up >= 0 && (q >> (up & 31)) == lane;
    const uint32_t pk = xlane(lane >> 1, t0), pn = xlane(lane >> 1, n0);
    const bool parentMoves = on && lane > 1 && pk > t;
    const bool vacant = lane == q || t0 > t;
    const bool land = on && vacant && !parentMoves;
    if (q >= 64) {
      const uint32_t qk = rlane(t0, q >> 1), qn = rlane(n0, q >> 1);
      const bool here = lane == (q & 63);
      t1 = here ? (qk > t ? qk : t) : t1;
      n1 = here ? (qk > t ? qn : n) : n1;
    }
    t0 = parentMoves ? pk : (land ? t : t0);
    n0 = parentMoves ? pn : (land ? n : n0);
  }
  BPSX_DEV void push(uint32_t t, uint32_t n, int lane) {
    size++;
    bubble_up(size, t, n, lane);
  }
  // dtNodeQueue::modify: the entry of node n (packed like n0) gets key t and bubbles up
  BPSX_DEV void modify(uint32_t n, uint32_t t, int lane) {
    const unsigned long long m0 = __ballot(lane >= 1 && lane <= size && n0 == n);
    const unsigned long long m1 = m0 ? 0ull : __ballot(64 + lane <= size && n1 == n);
    if (!(m0 | m1)) return;
    const int q = m0 ? __ffsll((long long)m0) - 1 : 64 + __ffsll((long long)m1) - 1;
    bubble_up(q, t, n, lane);
  }
  // dtNodeQueue::pop after the caller has taken the root.  The reference moves the hole left
  // by the root down to a leaf along the smaller children and then bubbles the former last
  // entry up from there; along that route keys never decrease, so the entry ends up above
  // the first route element greater than it and nothing below moves.  Which child the hole
  // moves to depends only on the children's keys, which the moves above them do not change:
  // every lane q picks the smaller child of position q (cross-lane reads; positions past the
  // end hold kEmpty), the route is read off that table with dependent lane reads, and then
  // every route position whose smaller child is not greater than the entry takes that child,
  // and the first one whose child is greater takes the entry.
  BPSX_DEV void pop(int lane) {
    const int last = size;
    size--;
    uint32_t lt, ln;
    if (last < 64) { lt = rlane(t0, last); ln = rlane(n0, last); t0 = wlane(t0, kEmpty, last); }
    else { lt = rlane(t1, last & 63); ln = rlane(n1, last & 63); t1 = wlane(t1, kEmpty, last & 63); }
    if (size == 0) return;
    const bool wide = size >= 64;           // entries in the second pair
    const bool lo = lane < 32;              // children of positions 32..63 are in the second pair
    const int c0 = (2 * lane) & 63;
    // keys and nodes of both children in one round of cross-lane reads
    uint32_t cl = xlane(c0, t0), cr = xlane(c0 + 1, t0);
    uint32_t nl = xlane(c0, n0), nr = xlane(c0 + 1, n0);
    if (wide) {
      const uint32_t hl = xlane(c0, t1), hr = xlane(c0 + 1, t1), ml = xlane(c0, n1), mr = xlane(c0 + 1, n1);
      cl = lo ? cl : hl; cr = lo ? cr : hr; nl = lo ? nl : ml; nr = lo ? nr : mr;
    } else {
      cl = lo ? cl : kEmpty; cr = lo ? cr : kEmpty;
    }
    const bool right = cr < cl;
    const uint32_t cmin = right ? cr : cl;
    const uint32_t cn = right ? nr : nl;
    const uint32_t choice = (uint32_t)(2 * lane) + (right ? 1u : 0u);   // position 2..127
    // route of the hole: 1, choice[1], choice[choice[1]], ...
    unsigned long long route = 2ull;
    uint32_t q = 1;
#pragma unroll
    for (int lvl = 0; lvl < 5; ++lvl) {
      q = rlane(choice, (int)(q & 31));     // levels 0..4 start from positions below 32
      route |= 1ull << (q & 63);
    }
    const bool on = (route >> lane) & 1ull;
    const bool take = on && cmin <= lt;
    const bool land = on && !take && (lane == 1 || t0 <= lt);
    if (wide) {
      // sixth level: from position q in 32..63 to its smaller child in the second pair, which has
      // no children of its own: it takes the entry if its parent took it
      const uint32_t e = rlane(choice, (int)(q & 63));
      const bool here = lane == (int)(e & 63) && t1 <= lt;
      t1 = here ? lt : t1;
      n1 = here ? ln : n1;
    }
    t0 = take ? cmin : (land ? lt : t0);
    n0 = take ? cn : (land ? ln : n0);
  }
};

// The open list as an unordered set in registers.  dtNodeQueue::pop returns the entry with the
// smallest total; while that smallest total is held by one entry only, which entry that is does
// not depend on how the binary heap happens to be arranged, so a set with a minimum search gives
// the same sequence of pops as the heap, at a fraction of its cost.  Entry p (0-based, dense:
// entries 0..size-1) lives in lane p & 63 of register pair p >> 6; unused places hold kEmpty
// keys and kNoNode nodes.  The minimum is found with a cross-lane reduction; push appends,
// modify rewrites the key of the entry that names the node, pop moves the last entry into the
// gap.  All writes are lane-predicated vector selects: no branches, no scalar lane writes.
// When two entries share the smallest total the heap's arrangement decides; the search keeps a
// log of its open-list operations for that case (see OpLog).
struct OpenBag {
  static constexpr int kCap = 128;
  static constexpr uint32_t kEmpty = 0x7fffffffu;   // above +inf; every key stays below 2^31
  static constexpr uint32_t kNoNode = 0xffffffffu;  // no packed node looks like this (26 bits)
  uint32_t t0, t1;   // total bits
  uint32_t n0, n1;   // node index (bits 0-10) | the node's polygon index << 11
  int size;          // places in use: 0..size-1, of which `hole` (if >= 0) is vacant
  int hole;
  BPSX_DEV void init() { t0 = t1 = kEmpty; n0 = n1 = kNoNode; size = 0; hole = -1; }
  BPSX_DEV int count() const { return size - (hole >= 0 ? 1 : 0); }
  static BPSX_DEV uint32_t umin(uint32_t v, uint32_t w) { return w < v ? w : v; }
  // smallest key of the wavefront, as a wave-uniform value
  static BPSX_DEV uint32_t wave_min(uint32_t v) {
    // within rows of 16 lanes: exchange over 1, 2, mirror within 8, mirror within 16.  A lane
    // pattern on an operand needs two idle cycles after the write of that register.
    asm("s_nop 1\n\t"
        "v_min_u32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_min_u32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_min_u32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_min_u32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0"
        : "+v"(v));
    // every lane now holds its row's minimum: the four rows meet on the scalar unit
    const uint32_t a = rlane(v, 0), b = rlane(v, 16), c = rlane(v, 32), d = rlane(v, 48);
    const uint32_t ab = a < b ? a : b, cd = c < d ? c : d;
    return ab < cd ? ab : cd;
  }
  BPSX_DEV uint32_t key_at(int p) const {
    const uint32_t a = rlane(t0, p & 63), b = rlane(t1, p & 63);
    return p < 64 ? a : b;
  }
  BPSX_DEV uint32_t node_at(int p) const {
    const uint32_t a = rlane(n0, p & 63), b = rlane(n1, p & 63);
    return p < 64 ? a : b;
  }
  // Position of the entry with the smallest total and that total; *tie when another entry has
  // the same total.  The set must not be empty.
  BPSX_DEV int argmin(bool* tie, uint32_t* key) const {
    const uint32_t m = wave_min(umin(t0, t1));
    *key = m;
    const unsigned long long h0 = __ballot(t0 == m), h1 = __ballot(t1 == m);
    *tie = __popcll(h0) + __popcll(h1) > 1;
    return h0 ? __ffsll((long long)h0) - 1 : 64 + __ffsll((long long)h1) - 1;
  }
  // position of the entry of node `node` (packed like n0), or -1
  BPSX_DEV int find(uint32_t node) const {
    const unsigned long long h0 = __ballot(n0 == node && t0 != kEmpty), h1 = __ballot(n1 == node && t1 != kEmpty);
    return h0 ? __ffsll((long long)h0) - 1 : (h1 ? 64 + __ffsll((long long)h1) - 1 : -1);
  }
  BPSX_DEV void write(int p, uint32_t key, uint32_t node, int lane) {
    const int hi = lane + 64;
    t0 = lane == p ? key : t0;
    n0 = lane == p ? node : n0;
    t1 = hi == p ? key : t1;
    n1 = hi == p ? node : n1;
  }
  // takes entry p out; its place stays vacant until the next push fills it or settle() closes it
  BPSX_DEV void take(int p, int lane) {
    hole = p;
    t0 = lane == p ? kEmpty : t0;
    t1 = lane + 64 == p ? kEmpty : t1;
  }
  // ---- the set without order of places (astar_spec): an entry may sit anywhere, a vacant place
  // holds kEmpty; `size` counts the entries
  // adds an entry at the first vacant place; returns where
  BPSX_DEV int put(uint32_t key, uint32_t node, int lane) {
    const unsigned long long v0 = __ballot(t0 == kEmpty);
    int p;
    if (v0) p = __ffsll((long long)v0) - 1;
    else p = 64 + __ffsll((long long)__ballot(t1 == kEmpty)) - 1;
    size++;
    write(p, key, node, lane);
    return p;
  }
  // takes the entry at place p out
  BPSX_DEV void drop(int p, int lane) {
    size--;
    t0 = lane == p ? kEmpty : t0;
    t1 = lane + 64 == p ? kEmpty : t1;
  }
  // adds an entry; returns where
  BPSX_DEV int push(uint32_t key, uint32_t node, int lane) {
    int p;
    if (hole >= 0) { p = hole; hole = -1; }
    else { p = size; size = p + 1; }
    write(p, key, node, lane);
    return p;
  }
  // Closes a vacant place left at the end of an expansion: the last entry moves into it.
  // Returns the position the last entry had if it moved (so that the caller can follow it), else -1.
  BPSX_DEV int settle(int lane, int* to) {
    if (hole < 0) return -1;
    const int h = hole, last = size - 1;
    *to = h;
    hole = -1;
    size = last;
    if (h == last) return -1;   // the vacant place was the last one: its key is kEmpty already
    const uint32_t lt = key_at(last), ln = node_at(last);
    write(h, lt, ln, lane);
    t0 = lane == last ? kEmpty : t0;
    t1 = lane + 64 == last ? kEmpty : t1;
    return last;
  }
  // the entry of node `node` gets key `key`
  BPSX_DEV void modify(uint32_t node, uint32_t key) {
    t0 = (n0 == node && t0 != kEmpty) ? key : t0;
    t1 = (n1 == node && t1 != kEmpty) ? key : t1;
  }
};

// Log of a search's open-list operations, in the wavefront's HBM slot: what is needed to
// rebuild the reference's binary heap at the moment two open entries share the smallest total.
// Replaying the log through the exact heap (RegHeap) gives the heap's arrangement and with it
// the entry dtNodeQueue::pop would return; the search then carries on with the set, and the
// next tie replays only what was logged since.  word = packed node | op << 30.
constexpr uint32_t kOpPush = 0u, kOpModify = 1u, kOpPop = 2u;

struct AstarState {
  int lastBest;
  float lastBestCost;
  bool outOfNodes;
  RegHeap rh;
  OpenBag bag;
  int logPos;      // entries written to the operation log
  int logDone;     // entries of it already applied to rh
  // the entry that will be popped next: position, key and how many entries hold that key
  int nextPos, nextCount;
  uint32_t nextKey, nextNode;
  AEdge pf;        // edge records of polygon pfIp, requested ahead (lanes 0..5)
  uint32_t pfIp;
  // ---- two-at-a-time expansion (astar_spec): the smallest open entries wait in four slots,
  // slot s in lanes 8 s .. 8 s + 5, with their polygons' edge records already requested
  uint32_t fKey, fNode;     // per lane: key and packed node of the lane's slot (kEmpty: slot vacant)
  AEdge fe;                 // per lane: edge record (lane & 7) of the slot's polygon
  uint32_t bmKey, bmNode;   // smallest entry of the set (the open entries not in a slot) ...
  int bmPos, bmCount;       // ... its place, and how many entries hold that key (0: set empty)
  uint32_t forceNode;       // after a tie was resolved from the log: the node to expand next (kNoNode: none)
};
constexpr int kSlots = 4;
enum AstarExit { kAstarEmpty = 0, kAstarGoal = 1, kAstarGrowLinks = 2, kAstarGrowHeap = 3 };

// Applies entries [from, to) of the operation log to the exact heap.
BPSX_DEV void replay_log(RegHeap& rh, const OpLogEntry* log, int from, int to, int lane) {
  for (int base = from; base < to; base += 64) {
    OpLogEntry e{0u, 0u};
    if (base + lane < to) e = log[base + lane];
    const int n = to - base < 64 ? to - base : 64;
    for (int i = 0; i < n; ++i) {
      const uint32_t key = rlane(e.key, i), w = rlane(e.word, i);
      const uint32_t op = w >> 30, node = w & 0x3fffffffu;
      if (op == kOpPop) rh.pop(lane);
      else if (op == kOpPush) rh.push(key, node, lane);
      else rh.modify(node, key, lane);
    }
  }
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

}  // namespace bpsx
#endif  // BPSX_GEODESIC_COMMON_H

#ifndef BPSX_GEO_NS
#define BPSX_GEO_NS geo
#endif
namespace bpsx {
namespace BPSX_GEO_NS {

#ifndef BPSX_LINKS_LDS
#define BPSX_LINKS_LDS 1152
#endif
#ifndef BPSX_HEAP_LDS
#define BPSX_HEAP_LDS 32
#endif
#ifndef BPSX_WINDOW
#define BPSX_WINDOW 128
#endif
constexpr int kLinksLds = BPSX_LINKS_LDS;   // nodes whose link word is kept in LDS
constexpr int kHeapLds = BPSX_HEAP_LDS;     // entries of an open list that has left the registers kept in LDS (its top levels)
constexpr int kWindow = BPSX_WINDOW;        // most recent nodes whose position/cost/total are kept in LDS
#ifndef BPSX_HASH
#define BPSX_HASH 512
#endif
constexpr int kHashSize = BPSX_HASH;        // buckets of the node pool's hash table
static_assert((kWindow & (kWindow - 1)) == 0 && kWindow >= 2 * kNvp, "window must be a power of two");

// LDS of one wavefront.
struct GeoLds {
  uint16_t first[kHashSize];
  union {
    HeapEntry heap[kHeapLds];      // open list once it has left the registers
    uint16_t w_parent[kWindow];    // until then: 1-based parent index of the window's nodes
  };
  uint32_t n_link[kLinksLds];      // polygon index (bits 0-14) | flags (bits 15-16: 1 open, 2 closed) | next node of the hash chain << 20
  float w_total[kWindow];
  float w_cost[kWindow];
  float w_pos[3][kWindow];
};
// After A* its LDS is dead; the funnel reuses it for the corridor and its portals.  The
// corridor is written while the nodes' links are still being read: it lies over the hash
// heads, which are no longer needed by then.
struct FunnelLds {
  uint16_t corridor[kMaxPath];
  uint16_t pad[kHashSize - kMaxPath];
  float portals[kMaxPath][6];
};
static_assert(offsetof(FunnelLds, portals) == offsetof(GeoLds, heap), "corridor must overlay the hash heads only");
union GeoShared {
  GeoLds a;
  FunnelLds f;
};

// Accessors take the instantiation's spill switch S: with S false every node index is below
// kLinksLds and every heap index below kHeapLds, and no address-space branch is generated.
struct GeoWave {
  GeoLds* L;
  GeoSlot* ws;
  int lane;
  int heapSize;
  int nodeCount;
  uint32_t linkSpills, heapSpills;   // queries that left the LDS links / the register heap
  uint32_t tieRestarts;              // queries run again with the exact heap (open list or log outgrew the fast path)
  uint32_t tieReplays;               // ties resolved by replaying the operation log
  uint32_t prefetchHits;             // expansions whose edge records had been requested ahead
#ifdef BPSX_QUERY_TRACE
  uint32_t missTop, missNb, maxHeap;
#endif

  // ---------------------------------------------------------------- node pool
  template <bool S> BPSX_DEV uint32_t link(int i) const {
    if (!S || i < kLinksLds) return L->n_link[i];
    BPSX_KEEP_APART();
    const uint32_t v = ws->nodes[i].link;
    BPSX_KEEP_APART();
    return v;
  }
  template <bool S> BPSX_DEV void set_link(int i, uint32_t v) const {
    if (!S || i < kLinksLds) L->n_link[i] = v;
    else { BPSX_KEEP_APART(); ws->nodes[i].link = v; BPSX_KEEP_APART(); }
  }
  // node i still has its position/cost/total in LDS
  BPSX_DEV bool in_window(int i) const { return i >= nodeCount - kWindow; }
  static BPSX_DEV uint32_t hash(uint32_t ip) { return (__umul24(ip, 0x9e3779u) >> 9) & (kHashSize - 1); }
  BPSX_DEV void clear() {
    for (int i = lane; i < kHashSize; i += 64) L->first[i] = (uint16_t)kChainEnd;
    heapSize = 0;
    nodeCount = 0;
    wave_sync();
  }
  // Node index of polygon ip, or -1; *head receives the bucket's first node (what a new node of
  // this bucket links to) and *hlink the found node's link word (its flags).  Called by all
  // lanes (idle ones with valid = false): the chains are walked in step, one LDS access per
  // lane and round, until every lane has hit or run out.
  template <bool S> BPSX_DEV int find(bool valid, uint32_t ip, uint32_t bucket, uint32_t* head, uint32_t* hlink) const {
    uint32_t cur = L->first[bucket];
    if (!valid) cur = kChainEnd;
    *head = cur;
    int found = -1;
    uint32_t fl = 0;
    while (__ballot(cur != kChainEnd)) {
      const bool live = cur != kChainEnd;
      const uint32_t l = link<S>(live ? (int)cur : 0);
      const bool hit = live && link_id(l) == ip;
      found = hit ? (int)cur : found;
      fl = hit ? l : fl;
      cur = (live && !hit) ? link_next(l) : kChainEnd;
    }
    *hlink = fl;
    return found;
  }

  // ---------------------------------------------------------------- open list, once it has
  // left the registers (more than kRegHeap entries: rare)
  // The heap is walked with wave-uniform indices: every lane issues the same LDS access and the
  // values are moved to scalar registers, so the loops below branch on the scalar unit and cost
  // a handful of vector instructions per level.
  template <bool S> BPSX_DEV HeapEntry hget(int i) const {
    if (!S || i < kHeapLds) return L->heap[i];
    BPSX_KEEP_APART();
    const HeapEntry e = ws->heap_spill[i];
    BPSX_KEEP_APART();
    return e;
  }
  template <bool S> BPSX_DEV void hset(int i, float t, int n) const {
    const HeapEntry e{t, (uint32_t)n};
    if (!S || i < kHeapLds) L->heap[i] = e;   // all lanes store the same value to the same address
    else if (lane == 0) { BPSX_KEEP_APART(); ws->heap_spill[i] = e; BPSX_KEEP_APART(); }
  }
  // dtNodeQueue::bubbleUp from index i with entry (t, n)
  template <bool S> BPSX_DEV void bubble_up(int i, float t, int n) const {
    while (i > 0) {
      const int parent = (i - 1) >> 1;
      const HeapEntry pe = hget<S>(parent);
      const float pt = uniform_f(pe.total);
      if (!(pt > t)) break;
      hset<S>(i, pt, uniform_i((int)pe.node));
      i = parent;
    }
    hset<S>(i, t, n);
    wave_sync();
  }
  template <bool S> BPSX_DEV void push(float t, int n) {
    heapSize++;
    bubble_up<S>(heapSize - 1, t, n);
  }
  template <bool S> BPSX_DEV void modify(int n, float t) const {
    int found = -1;
    for (int base = 0; base < heapSize; base += 64) {
      const int i = base + lane;
      const unsigned long long m = __ballot(i < heapSize && (int)hget<S>(i).node == n);
      if (m) { found = base + (__ffsll((long long)m) - 1); break; }
    }
    if (found >= 0) bubble_up<S>(found, t, n);
  }
  // dtNodeQueue::pop (the caller has read the root). The reference moves the hole left by the
  // root down to a leaf along the smaller children and then bubbles the former last entry up
  // from there; along that route keys never decrease, so the entry ends up above the first
  // route element that is greater than it: the walk can stop there, nothing below moves.
  template <bool S> BPSX_DEV void pop() {
    heapSize--;
    const int size = heapSize;
    if (size == 0) return;
    const HeapEntry lastE = hget<S>(size);
    const float lt = uniform_f(lastE.total);
    const int ln = uniform_i((int)lastE.node);
    int i = 0;
    for (;;) {
      const int c = 2 * i + 1;
      if (c >= size) break;
      const bool two = c + 1 < size;
      // odd lanes fetch the right child, even lanes the left one: one LDS instruction
      const HeapEntry e = hget<S>(c + ((two && (lane & 1)) ? 1 : 0));
      const float t0 = lane_f(e.total, 0), t1 = lane_f(e.total, 1);
      const bool right = two && t0 > t1;
      const float tc = right ? t1 : t0;
      if (!(tc <= lt)) break;
      const int nc = right ? lane_i((int)e.node, 1) : lane_i((int)e.node, 0);
      hset<S>(i, tc, nc);
      i = c + (right ? 1 : 0);
    }
    hset<S>(i, lt, ln);
    wave_sync();
  }
};

// The expansion loop of findPath.  M = 3: open list as an unordered set in registers, all links
// in LDS; M = 4: the same, links may spill.  These two return kAstarTie when two open entries
// share the smallest total; the search then starts again with the exact heap: M = 0: heap in
// registers, all links in LDS; M = 1: heap in registers, links may spill; M = 2: heap in
// LDS/HBM, links may spill.  Returns kAstarGrow* before an expansion that could outgrow what
// its mode holds.
template <int M>
BPSX_DEV AstarExit astar_loop(GeoWave& g, AstarState& st, const AEdge* edges, uint32_t endIp, const float* endPos, uint32_t* pops
#ifdef BPSX_PHASE_TIMING
                              , unsigned long long* phase_acc, unsigned long long& phase_t0
#endif
                              ) {
  const int lane = g.lane;
  GeoLds* L = g.L;
  const float H_SCALE = 0.999f;
  const float e0 = endPos[0], e1 = endPos[1], e2 = endPos[2];
  endIp = (uint32_t)uniform_i((int)endIp);   // the same in all lanes: the goal test stays on the scalar unit
  constexpr bool S = M == 1 || M == 2 || M == 4;    // links and states may be in HBM
  constexpr bool SH = M == 2;   // open list in LDS/HBM
  constexpr bool BAG = M >= 3;  // open list as an unordered set
  RegHeap& rh = st.rh;
  OpenBag& bag = st.bag;
  while ((SH ? g.heapSize : (BAG ? bag.size : rh.size)) > 0) {   // (the set has no vacant place here: size is its count)
    if (!S && g.nodeCount > kLinksLds - kNvp) return kAstarGrowLinks;
    if (!SH && !BAG && rh.size > kRegHeap - kNvp) return kAstarGrowHeap;
    // the set, the heap that is rebuilt from the log on a tie, and the log itself must hold one more expansion
    if (BAG && (bag.size > kRegHeap - kNvp || st.logPos > kOpLogCap - 2 * kNvp)) return kAstarGrowHeap;
    // the node about to be popped is known before the open list is repaired: fetch its edges
    // meanwhile
    int bi;
    uint32_t bestIp;
    uint32_t blink;   // the node's link word: closing the node rewrites its flags
    int bagPos = 0;
    if (BAG) {
      // The smallest entry is known from the end of the previous expansion: the runner-up found
      // then, unless a key written since is smaller (st.next*).
      bagPos = st.nextPos;
      uint32_t root;
      if (st.nextCount > 1) {
        // two open entries share the smallest total: the reference's heap decides.  Bring the
        // exact heap up to date from the log; its root is the entry to pop.
        wave_sync();
        replay_log(rh, g.ws->oplog, st.logDone, st.logPos, lane);
        st.logDone = st.logPos;
        g.tieReplays++;
        root = rlane(rh.n0, 1);
        bagPos = bag.find(root);
      } else {
        root = st.nextNode;
      }
      bi = (int)(root & 0x7ffu);
      bestIp = root >> 11;
      blink = g.link<S>(bi);
    } else if (SH) {
      bi = uniform_i((int)L->heap[0].node);
      blink = g.link<S>(bi);
      bestIp = link_id((uint32_t)uniform_i((int)blink));
    } else {
      const uint32_t root = rlane(rh.n0, 1);
      bi = (int)(root & 0x7ffu);
      bestIp = root >> 11;
      blink = g.link<S>(bi);
    }
    uint32_t nb = kNoNb;
    float m0 = 0, m1 = 0, m2 = 0;
    // its edge records were requested one expansion ago if it was the runner-up then
    const bool prefetched = BAG && bestIp == st.pfIp;
    if (prefetched) {
      nb = st.pf.nb; m0 = st.pf.mid[0]; m1 = st.pf.mid[1]; m2 = st.pf.mid[2];
      if (lane >= kNvp) nb = kNoNb;
      g.prefetchHits++;
    } else if (lane < kNvp) {
      const AEdge e = edges[bestIp * kNvp + lane];
      nb = e.nb; m0 = e.mid[0]; m1 = e.mid[1]; m2 = e.mid[2];
    }
    float b0, b1, b2, bcost;
    uint32_t bparent;   // read now, moved to a scalar register only after the pop
    if (g.in_window(bi)) {
      const int w = bi & (kWindow - 1);
      b0 = L->w_pos[0][w]; b1 = L->w_pos[1][w]; b2 = L->w_pos[2][w]; bcost = L->w_cost[w];
      if (!SH) bparent = L->w_parent[w];
      else { BPSX_KEEP_APART(); bparent = g.ws->nodes[bi].parent; BPSX_KEEP_APART(); }
    } else {
      BPSX_KEEP_APART();
      const float4 pc = *reinterpret_cast<const float4*>(g.ws->nodes[bi].pos);   // pos, cost
      b0 = pc.x; b1 = pc.y; b2 = pc.z; bcost = pc.w;
      bparent = g.ws->nodes[bi].parent;
      BPSX_KEEP_APART();
#ifdef BPSX_QUERY_TRACE
      g.missTop++;
#endif
    }
#ifdef BPSX_QUERY_TRACE
    if (!SH && (uint32_t)rh.size > g.maxHeap) g.maxHeap = (uint32_t)rh.size;
#endif
    PHASE_MARK(0);
    if (BAG) {
      bag.take(bagPos, lane);
      // the smallest of what remains is the next node to expand unless this expansion writes a
      // smaller key: note it, and request its polygon's edge records now
      st.nextCount = 0;
      st.pfIp = kNoNb;
      if (bag.size > 1) {
        bool tie;
        st.nextPos = bag.argmin(&tie, &st.nextKey);
        st.nextCount = tie ? 2 : 1;
        st.nextNode = bag.node_at(st.nextPos);
        st.pfIp = st.nextNode >> 11;
        if (lane < kNvp) st.pf = edges[st.pfIp * kNvp + lane];
      }
    }
    else if (SH) g.pop<true>();
    else rh.pop(lane);
    const uint32_t pidx = (uint32_t)uniform_i((int)bparent);
    PHASE_MARK(1);
    g.set_link<S>(bi, with_flags(blink, 2u));   // open -> closed
    if (bestIp == endIp) { st.lastBest = bi; return kAstarGoal; }
    (*pops)++;
    PHASE_MARK(2);
    const uint32_t bucket = GeoWave::hash(nb);
    uint32_t chainHead, hitLink;
    int ni = g.find<S>(nb != kNoNb, nb, bucket, &chainHead, &hitLink);
    // the polygon the expanded node was reached from is not entered again
    if (pidx && ni + 1 == (int)pidx) nb = kNoNb;
    PHASE_MARK(3);
    // new nodes take consecutive indices in edge order; past the pool's end they are dropped
    const bool isNew = nb != kNoNb && ni < 0;
    const unsigned long long need = __ballot(isNew);
    if (need) {
      const int rank = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(need >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)need, 0u));
      const int count = __popcll(need);
      if (isNew) {
        const int idx = g.nodeCount + rank;
        if (!S || idx < kMaxNodes) ni = idx;
        else nb = kNoNb;
      }
      const int want = g.nodeCount + count;
      // the reference carries on without the dropped nodes, but reports anything found after
      // that as failure (only plain DT_SUCCESS counts, PathFinder.cpp:506): the search can stop
      if (S && want > kMaxNodes) { st.outOfNodes = true; return kAstarEmpty; }
      g.nodeCount = (!S || want < kMaxNodes) ? want : kMaxNodes;
      bool pending = isNew && nb != kNoNb;
      // All insert at once in front of the chain head their lookup saw.  Of several that share a
      // bucket one store wins; the others see that when they read the head back and go round
      // again behind the winner.  One new node needs no check.  A new node is open from the
      // start: the cost computation below always takes it.
      uint32_t head = chainHead;
      for (;;) {
        if (pending) {
          g.set_link<S>(ni, make_link(nb, 1u, head));
          L->first[bucket] = (uint16_t)ni;
        }
        wave_sync();
        if (count == 1) break;
        if (pending) {
          head = L->first[bucket];
          pending = head != (uint32_t)ni;
        }
        wave_sync();
        if (!__ballot(pending)) break;
      }
    }
    PHASE_MARK(4);
#ifdef BPSX_QUERY_TRACE
    g.missNb += (uint32_t)__popcll(__ballot(nb != kNoNb && !isNew && !g.in_window(ni)));
#endif
    // Costs of the step to each neighbour (lane-wise).  Written with few branches: all lanes
    // issue the one round of LDS reads a revisited node needs (idle lanes read slot 0; its flags
    // came with the lookup), the rare node that has left the window is fetched under a
    // wave-uniform test, new nodes take the portal midpoint instead, and everything is stored
    // in one predicated block.
    const bool valid = nb != kNoNb;
    const int nis = valid ? ni : 0;
    const int w = nis & (kWindow - 1);
    const bool inw = g.in_window(nis);   // new nodes always are
    ANode& hn = g.ws->nodes[nis];
    uint32_t fl = link_flags(hitLink);
    float p0 = L->w_pos[0][w], p1 = L->w_pos[1][w], p2 = L->w_pos[2][w], oldTotal = L->w_total[w];
    const bool miss = valid && !isNew && !inw;
    if (__ballot(miss)) {
      if (miss) {
        BPSX_KEEP_APART();
        const float4 pc = *reinterpret_cast<const float4*>(hn.pos);     // pos, cost
        p0 = pc.x; p1 = pc.y; p2 = pc.z; oldTotal = hn.total;
        BPSX_KEEP_APART();
      }
    }
    if (isNew) { p0 = m0; p1 = m1; p2 = m2; fl = 0; }
    // both square roots in one pass: lanes 8..13 take the second operand of lanes 0..5
    const float cx = p0 - b0, cy = p1 - b1, cz = p2 - b2;
    const float ex = e0 - p0, ey = e1 - p1, ez = e2 - p2;
    const float cc = cx * cx + cy * cy + cz * cz, ee = ex * ex + ey * ey + ez * ez;
    const float roots = sqrt_exact(lanes_up8(cc, ee));
    const float curCost = roots * 1.0f;
    const float toEnd = lanes_down8(roots);
    const bool last = nb == endIp;
    const float cost = last ? bcost + curCost + toEnd * 1.0f : bcost + curCost;
    const float heuristic = last ? 0.0f : toEnd * H_SCALE;
    const float total = cost + heuristic;
    const bool update = valid && !(fl && total >= oldTotal);
    const bool wasOpen = update && (fl & 1u) != 0;
    if (update) {
      if (!isNew) g.set_link<S>(ni, with_flags(hitLink, 1u));   // open (again)
      if (inw) {
        L->w_pos[0][w] = p0; L->w_pos[1][w] = p1; L->w_pos[2][w] = p2;   // unchanged for a revisited node
        L->w_cost[w] = cost; L->w_total[w] = total;
        if (!SH) L->w_parent[w] = (uint16_t)(bi + 1);
      }
      *reinterpret_cast<float4*>(hn.pos) = make_float4(p0, p1, p2, cost);
      *reinterpret_cast<uint2*>(&hn.total) = make_uint2(__float_as_uint(total), (uint32_t)(bi + 1));   // total, parent = expanded node
    }
    wave_sync();
    PHASE_MARK(5);
    // ---- ordered phase, in edge order.  First the "nearest so far" record (lastBestNode of
    // findPath): an update replaces it when its heuristic is lower; only lanes below the
    // current record can matter, usually none.
    const uint32_t packed = (uint32_t)ni | (nb << 11);   // heap entry of this lane's node
    unsigned long long better = __ballot(update && heuristic < st.lastBestCost);
    while (better) {
      const int src = __ffsll((long long)better) - 1;
      better &= better - 1;
      const float h = lane_f(heuristic, src);
      if (h < st.lastBestCost) { st.lastBestCost = h; st.lastBest = (int)(rlane(packed, src) & 0x7ffu); }
    }
    // then the open list
    unsigned long long upd = __ballot(update);
    const unsigned long long openMask = __ballot(wasOpen);
    if (BAG) {
      // log: this expansion's pop (written by lane 63, which handles no edge), then its updates in edge order
      const int rank = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(upd >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)upd, 0u));
      if (update || lane == 63) {
        OpLogEntry e;
        e.key = __float_as_uint(total);
        e.word = update ? (packed | ((wasOpen ? kOpModify : kOpPush) << 30)) : (kOpPop << 30);
        g.ws->oplog[st.logPos + (update ? 1 + rank : 0)] = e;
      }
      st.logPos += 1 + __popcll(upd);
    }
    while (upd) {
      const int src = __ffsll((long long)upd) - 1;
      upd &= upd - 1;
      const uint32_t entry = rlane(packed, src);
      const float t = lane_f(total, src);
      const bool open = (openMask >> src) & 1ull;
      if (BAG) {
        const uint32_t key = __float_as_uint(t);
        int at;
        if (open) { at = bag.find(entry); bag.modify(entry, key); }
        else at = bag.push(key, entry, lane);
        if (st.nextCount != 0 && at == st.nextPos) {
          st.nextKey = key; st.nextCount = 1;   // the smallest entry itself got a smaller key
        } else if (key < st.nextKey || st.nextCount == 0) {
          st.nextKey = key; st.nextPos = at; st.nextCount = 1; st.nextNode = entry;
        } else if (key == st.nextKey) {
          st.nextCount++;
        }
      } else if (SH) {
        if (open) g.modify<true>((int)(entry & 0x7ffu), t);
        else g.push<true>(t, (int)(entry & 0x7ffu));
      } else {
        if (open) rh.modify(entry, __float_as_uint(t), lane);
        else rh.push(__float_as_uint(t), entry, lane);
      }
    }
    if (BAG) {
      // no push took the popped entry's place: close it, and follow the smallest entry if it is the one that moves
      int to = 0;
      const int moved = bag.settle(lane, &to);
      if (moved >= 0 && st.nextCount != 0 && st.nextPos == moved) st.nextPos = to;
    }
    PHASE_MARK(6);
  }
  return kAstarEmpty;
}

// The expansion loop of findPath, two nodes at a time.
//
// The reference expands one node per iteration: the open node with the smallest total.  Here the
// two smallest (A, then B) are worked on by the same instructions in different lanes: edge
// records, node lookup and costs of both are computed together, without side effects, from the
// state before either expansion.  A's results are then committed.  B's results are what the
// reference would compute after A's expansion, and are committed too, if
//   - B is still the node the reference would pop next: none of A's updates has a total at or
//     below B's, and no other open entry shares B's total,
//   - nothing B looked at was changed by A: B evaluates no polygon that A evaluates, not A's own
//     polygon, and A does not evaluate B's polygon,
//   - B is not the goal, and the node pool has room for both.
// Otherwise B simply stays where it is and is A in the next iteration.  On the benchmark's
// scenes three iterations out of four commit both, which nearly halves the instructions per
// expanded node: a search is one chain of dependent instructions, and its length, not memory
// bandwidth, sets the time of the longest searches and of the launch.
//
// The open entries live in a register set (OpenBag); the smallest ones are moved ahead of time
// into four slots (lanes 8 s .. 8 s + 5) whose polygons' edge records are requested at once, so
// that they have arrived when the slot's turn comes.  Ties for the smallest total are resolved
// by replaying the operation log through the exact heap, as the order then depends on the
// heap's arrangement.  S: node links may be in HBM (more than kLinksLds nodes).
template <bool S>
BPSX_DEV AstarExit astar_spec(GeoWave& g, AstarState& st, const AEdge* edges, uint32_t endIp, const float* endPos, uint32_t* pops
#ifdef BPSX_PHASE_TIMING
                              , unsigned long long* phase_acc, unsigned long long& phase_t0
#endif
                              ) {
  const int lane = g.lane;
  GeoLds* L = g.L;
  const float H_SCALE = 0.999f;
  const float e0 = endPos[0], e1 = endPos[1], e2 = endPos[2];
  endIp = (uint32_t)uniform_i((int)endIp);
  const int slot = lane >> 3, el = lane & 7;
  const bool edgeLane = slot < kSlots && el < kNvp;
  OpenBag& bag = st.bag;
  RegHeap& rh = st.rh;
  constexpr uint32_t kE = OpenBag::kEmpty;

  // the set's smallest entry, after its contents changed in ways the running record does not follow
  auto rescan = [&]() {
    st.bmCount = 0;
    if (bag.size > 0) {
      bool tie;
      st.bmPos = bag.argmin(&tie, &st.bmKey);
      st.bmCount = tie ? 2 : 1;
      st.bmNode = bag.node_at(st.bmPos);
    }
  };
  // an entry enters the set: keep the record of the smallest
  auto bag_push = [&](uint32_t key, uint32_t node) {
    const int at = bag.put(key, node, lane);
    if (st.bmCount == 0 || key < st.bmKey) { st.bmKey = key; st.bmPos = at; st.bmNode = node; st.bmCount = 1; }
    else if (key == st.bmKey) st.bmCount++;
  };
  // the set's entry at `pos` moves into slot s, and its polygon's edge records are requested
  auto bring = [&](int pos, uint32_t key, uint32_t node, int s) {
    bag.drop(pos, lane);
    if (slot == s) { st.fKey = key; st.fNode = node; }
    if (slot == s && el < kNvp) st.fe = edges[(node >> 11) * kNvp + (uint32_t)el];
    rescan();
  };

  // Every pass either expands a node or moves an entry into a slot; a search expands a few thousand
  // nodes at most.  The bound only guards against an endless loop should the bookkeeping ever
  // be inconsistent: the caller then runs the search again on the plain path.
  for (int pass = 0;; ++pass) {
    if (pass > 16 * kMaxNodes) return kAstarGrowHeap;
    // room for two more expansions in whatever is bounded
    if (!S && g.nodeCount > kLinksLds - 2 * kNvp) return kAstarGrowLinks;
    if (bag.size + kSlots > kRegHeap - 2 * kNvp || st.logPos > kOpLogCap - 4 * kNvp) return kAstarGrowHeap;
    // ---- the slots' keys, and the smallest three of them (a tournament of four)
    const uint32_t k0 = rlane(st.fKey, 0), k1 = rlane(st.fKey, 8), k2 = rlane(st.fKey, 16), k3 = rlane(st.fKey, 24);
    uint32_t ka, kb, kc;
    int sa, sb;
    {
      const bool c01 = k1 < k0, c23 = k3 < k2;
      const uint32_t a01 = c01 ? k1 : k0, b01 = c01 ? k0 : k1, a23 = c23 ? k3 : k2, b23 = c23 ? k2 : k3;
      const int i01 = c01 ? 1 : 0, j01 = c01 ? 0 : 1, i23 = c23 ? 3 : 2, j23 = c23 ? 2 : 3;
      const bool cf = a23 < a01;
      ka = cf ? a23 : a01; sa = cf ? i23 : i01;
      const uint32_t lf = cf ? a01 : a23, ls = cf ? b23 : b01;     // the final's loser, the winner's semi-final loser
      const int ilf = cf ? i01 : i23, ils = cf ? j23 : j01;
      const bool cs = ls < lf;
      kb = cs ? ls : lf; sb = cs ? ils : ilf;
      const uint32_t r1 = cs ? lf : ls, r2 = cf ? b01 : b23;
      kc = r2 < r1 ? r2 : r1;
    }
    const bool bagHas = st.bmCount > 0;
    if (ka == kE && !bagHas) return kAstarEmpty;   // nothing open any more
    if (st.forceNode == OpenBag::kNoNode) {
      // the smallest open entry must be in a slot: it may be in the set instead (an entry written
      // by the last expansion, or the slots have just been emptied)
      if (bagHas && (ka == kE || st.bmKey < ka)) {
        if (st.bmCount > 1) {
          // ... and shares its total with another entry of the set: the heap decides (below)
          ka = st.bmKey;
        } else {
          int s = k0 == kE ? 0 : (k1 == kE ? 1 : (k2 == kE ? 2 : (k3 == kE ? 3 : -1)));
          if (s < 0) {
            // every slot is taken: the one with the largest total goes back to the set
            uint32_t kw = k0; s = 0;
            if (k1 > kw) { kw = k1; s = 1; }
            if (k2 > kw) { kw = k2; s = 2; }
            if (k3 > kw) { kw = k3; s = 3; }
            const int keep = st.bmPos;      // places do not move when an entry is added
            const uint32_t kk = st.bmKey, kn = st.bmNode;
            bag_push(kw, rlane(st.fNode, s * 8));
            bring(keep, kk, kn, s);
          } else {
            bring(st.bmPos, st.bmKey, st.bmNode, s);
          }
          continue;
        }
      }
      // is the smallest total held by one entry only?
      const bool tie = kb == ka || (bagHas && st.bmKey == ka);
      if (tie) {
        // The reference's heap decides.  Bring the exact heap up to date from the log; its
        // root is the entry to pop.
        wave_sync();
        replay_log(rh, g.ws->oplog, st.logDone, st.logPos, lane);
        st.logDone = st.logPos;
        g.tieReplays++;
        st.forceNode = rlane(rh.n0, 1);
        continue;
      }
    } else {
      // the node the exact heap named: in a slot, or to be moved to one
      const uint32_t want = st.forceNode;
      const uint32_t n0 = rlane(st.fNode, 0), n1 = rlane(st.fNode, 8), n2 = rlane(st.fNode, 16), n3 = rlane(st.fNode, 24);
      sa = (k0 != kE && n0 == want) ? 0 : ((k1 != kE && n1 == want) ? 1 : ((k2 != kE && n2 == want) ? 2 : ((k3 != kE && n3 == want) ? 3 : -1)));
      if (sa < 0) {
        int s = k0 == kE ? 0 : (k1 == kE ? 1 : (k2 == kE ? 2 : (k3 == kE ? 3 : -1)));
        const int pos = bag.find(want);
        if (pos < 0) return kAstarGrowHeap;   // cannot happen: the heap's root is an open entry
        if (s < 0) {
          uint32_t kw = k0; s = 0;
          if (k1 > kw) { kw = k1; s = 1; }
          if (k2 > kw) { kw = k2; s = 2; }
          if (k3 > kw) { kw = k3; s = 3; }
          bag_push(kw, rlane(st.fNode, s * 8));
        }
        bring(pos, bag.key_at(pos), want, s);
        continue;
      }
      ka = rlane(st.fKey, sa * 8);
    }
    const bool forced = st.forceNode != OpenBag::kNoNode;
    st.forceNode = OpenBag::kNoNode;
    // ---- A is slot sa.  B: the smallest of the other slots, if it is the second smallest open entry.
    const uint32_t nodeA = rlane(st.fNode, sa * 8);
    const int biA = (int)(nodeA & 0x7ffu);
    const uint32_t ipA = nodeA >> 11;
    if (forced) {
      // (the forced slot need not hold the smallest key of the slots' tournament: find the runner-up anew)
      kb = kE; sb = 0; kc = kE;
    }
    const uint32_t nodeB = rlane(st.fNode, sb * 8);
    const uint32_t ipB = nodeB >> 11;
    if (ipA == endIp) {
      // the goal is popped: closed, not expanded
      if (lane == 0) g.set_link<S>(biA, with_flags(g.link<S>(biA), 2u));
      st.lastBest = biA;
      return kAstarGoal;
    }
    const bool spec = !forced && kb != kE && kc != kb && kb > ka && (!bagHas || kb < st.bmKey) && ipB != endIp &&
                      (!S || g.nodeCount + 2 * kNvp <= kMaxNodes);
    PHASE_MARK(0);
    // ---- slots vacated by the last pass take the set's smallest entries now: their polygons'
    // edge records are on the way while this pass works on A and B (whose records are taken
    // out of the slot registers first, so that nothing below waits for the new requests)
    const AEdge cur = st.fe;
    const uint32_t curNode = st.fNode;
    if (st.bmCount > 0 && k0 == kE) bring(st.bmPos, st.bmKey, st.bmNode, 0);
    if (st.bmCount > 0 && k1 == kE) bring(st.bmPos, st.bmKey, st.bmNode, 1);
    if (st.bmCount > 0 && k2 == kE) bring(st.bmPos, st.bmKey, st.bmNode, 2);
    if (st.bmCount > 0 && k3 == kE) bring(st.bmPos, st.bmKey, st.bmNode, 3);
    PHASE_MARK(1);
    // ---- both expansions, lane-wise, without side effects
    const bool inA = slot == sa, inB = spec && slot == sb;
    const bool act = edgeLane && (inA || inB);
    const int bi = (int)(curNode & 0x7ffu);       // the lane's slot's node
    uint32_t nb = act ? cur.nb : kNoNb;
    const float m0 = cur.mid[0], m1 = cur.mid[1], m2 = cur.mid[2];
    // the expanded nodes' own position, cost and parent
    float b0, b1, b2, bcost;
    uint32_t pidx;
    {
      const int bis = act ? bi : 0;
      const int w = bis & (kWindow - 1);
      b0 = L->w_pos[0][w]; b1 = L->w_pos[1][w]; b2 = L->w_pos[2][w]; bcost = L->w_cost[w];
      pidx = L->w_parent[w];
      const bool gone = act && !g.in_window(bis);
      if (__ballot(gone)) {
        if (gone) {
          BPSX_KEEP_APART();
          const float4 pc = *reinterpret_cast<const float4*>(g.ws->nodes[bis].pos);   // pos, cost
          b0 = pc.x; b1 = pc.y; b2 = pc.z; bcost = pc.w;
          pidx = g.ws->nodes[bis].parent;
          BPSX_KEEP_APART();
        }
      }
    }
    const uint32_t bucket = GeoWave::hash(nb);
    uint32_t chainHead, hitLink;
    int ni = g.find<S>(nb != kNoNb, nb, bucket, &chainHead, &hitLink);
    // the polygon the expanded node was reached from is not entered again
    if (pidx && ni + 1 == (int)pidx) nb = kNoNb;
    PHASE_MARK(2);
    const bool valid = nb != kNoNb;
    const bool isNew = valid && ni < 0;
    float p0, p1, p2, oldTotal;
    uint32_t fl = link_flags(hitLink);
    {
      const int nis = (valid && !isNew) ? ni : 0;
      const int w = nis & (kWindow - 1);
      p0 = L->w_pos[0][w]; p1 = L->w_pos[1][w]; p2 = L->w_pos[2][w]; oldTotal = L->w_total[w];
      const bool miss = valid && !isNew && !g.in_window(nis);
      if (__ballot(miss)) {
        if (miss) {
          BPSX_KEEP_APART();
          const ANode& hn = g.ws->nodes[nis];
          const float4 pc = *reinterpret_cast<const float4*>(hn.pos);
          p0 = pc.x; p1 = pc.y; p2 = pc.z; oldTotal = hn.total;
          BPSX_KEEP_APART();
        }
      }
    }
    if (isNew) { p0 = m0; p1 = m1; p2 = m2; fl = 0; }
    const float cx = p0 - b0, cy = p1 - b1, cz = p2 - b2;
    const float ex = e0 - p0, ey = e1 - p1, ez = e2 - p2;
    const float curCost = sqrt_exact(cx * cx + cy * cy + cz * cz) * 1.0f;
    const float toEnd = sqrt_exact(ex * ex + ey * ey + ez * ez);
    const bool last = nb == endIp;
    const float cost = last ? bcost + curCost + toEnd * 1.0f : bcost + curCost;
    const float heuristic = last ? 0.0f : toEnd * H_SCALE;
    const float total = cost + heuristic;
    const bool update = valid && !(fl && total >= oldTotal);
    const bool wasOpen = update && (fl & 1u) != 0;
    PHASE_MARK(3);
    // ---- may B be committed after A?
    bool commitB = spec;
    if (spec) {
      // A's new totals all lie above B's, so that B stays the next to pop
      if (__ballot(inA && update && __float_as_uint(total) <= kb)) commitB = false;
      // B evaluates A's polygon, or A evaluates B's
      if (__ballot((inB && nb == ipA) || (inA && nb == ipB))) commitB = false;
      // a polygon both evaluate
      unsigned long long both = 0;
#pragma unroll
      for (int j = 0; j < kNvp; ++j) {
        const uint32_t aj = rlane(nb, sa * 8 + j);
        both |= __ballot(inB && nb == aj && aj != kNoNb);
      }
      if (both) commitB = false;
    }
    PHASE_MARK(4);
    // ---- commit: A's results, and B's behind them
    if (commitB) g.prefetchHits++;
    const bool mine = inA || (commitB && inB);
    const unsigned long long mA = 0x3full << (sa * 8), mB = commitB ? 0x3full << (sb * 8) : 0ull;
    *pops += commitB ? 2u : 1u;
    if (lane == sa * 8 || (commitB && lane == sb * 8)) g.set_link<S>(bi, with_flags(g.link<S>(bi), 2u));   // open -> closed
    // new nodes take consecutive indices in edge order, A's before B's; past the pool's end the search stops
    const bool newM = mine && isNew;
    const unsigned long long need = __ballot(newM);
    if (need) {
      const unsigned long long needA = need & mA, needB = need & mB;
      const int cntA = __popcll(needA), count = __popcll(need);
      const int rank = inA ? (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(needA >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)needA, 0u))
                           : cntA + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(needB >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)needB, 0u));
      const int want = g.nodeCount + count;
      // the reference carries on without the dropped nodes, but reports anything found after
      // that as failure (only plain DT_SUCCESS counts, PathFinder.cpp:506): the search can stop
      if (S && want > kMaxNodes) { st.outOfNodes = true; return kAstarEmpty; }
      if (newM) ni = g.nodeCount + rank;
      g.nodeCount = want;
      // All insert at once in front of the chain head their lookup saw (the state before either
      // expansion).  Of several that share a bucket one store wins; the others see that when
      // they read the head back and go round again behind the winner.
      uint32_t head = chainHead;
      bool pending = newM;
      for (;;) {
        if (pending) {
          g.set_link<S>(ni, make_link(nb, 1u, head));
          L->first[bucket] = (uint16_t)ni;
        }
        wave_sync();
        if (count == 1) break;
        if (pending) {
          head = L->first[bucket];
          pending = head != (uint32_t)ni;
        }
        wave_sync();
        if (!__ballot(pending)) break;
      }
    }
    const bool upd = mine && update;
    if (upd) {
      if (!isNew) g.set_link<S>(ni, with_flags(hitLink, 1u));   // open (again)
      const int w = ni & (kWindow - 1);
      if (g.in_window(ni)) {     // with the pool as it is now: an old node may just have left the window
        L->w_pos[0][w] = p0; L->w_pos[1][w] = p1; L->w_pos[2][w] = p2;
        L->w_cost[w] = cost; L->w_total[w] = total;
        L->w_parent[w] = (uint16_t)(bi + 1);
      }
      ANode& hn = g.ws->nodes[ni];
      *reinterpret_cast<float4*>(hn.pos) = make_float4(p0, p1, p2, cost);
      *reinterpret_cast<uint2*>(&hn.total) = make_uint2(__float_as_uint(total), (uint32_t)(bi + 1));
    }
    wave_sync();
    PHASE_MARK(5);
    // the "nearest so far" record (lastBestNode of findPath): A's updates in edge order, then B's
    const uint32_t packed = (uint32_t)ni | (nb << 11);
    {
      const unsigned long long better = __ballot(upd && heuristic < st.lastBestCost);
      if (better) {
        unsigned long long part[2] = {better & mA, better & mB};
#pragma unroll
        for (int t = 0; t < 2; ++t)
          while (part[t]) {
            const int src = __ffsll((long long)part[t]) - 1;
            part[t] &= part[t] - 1;
            const float h = lane_f(heuristic, src);
            if (h < st.lastBestCost) { st.lastBestCost = h; st.lastBest = (int)(rlane(packed, src) & 0x7ffu); }
          }
      }
    }
    // log: A's pop (written by lane 63, which handles no edge), A's updates in edge order, then
    // B's pop (lane 62) and updates
    unsigned long long um = __ballot(upd);
    const unsigned long long openMask = __ballot(upd && wasOpen);
    {
      const unsigned long long umA = um & mA, umB = um & mB;
      const int cuA = __popcll(umA);
      const int at = inA ? 1 + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(umA >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)umA, 0u))
                         : 2 + cuA + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(umB >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)umB, 0u));
      if (upd || lane == 63 || (commitB && lane == 62)) {
        OpLogEntry e;
        e.key = __float_as_uint(total);
        e.word = upd ? (packed | ((wasOpen ? kOpModify : kOpPush) << 30)) : (kOpPop << 30);
        g.ws->oplog[st.logPos + (upd ? at : (lane == 63 ? 0 : 1 + cuA))] = e;
      }
      st.logPos += (commitB ? 2 : 1) + __popcll(um);
    }
    PHASE_MARK(6);
    // the expanded nodes' slots are vacant now
    if (mine) st.fKey = kE;
    // the open entries: a node already open is in a slot or in the set
    while (um) {
      const int src = __ffsll((long long)um) - 1;
      um &= um - 1;
      const uint32_t entry = rlane(packed, src);
      const uint32_t key = __float_as_uint(lane_f(total, src));
      if ((openMask >> src) & 1ull) {
        // in a slot?  (a slot just vacated keeps its old node: that one is closed, and a closed node is pushed, not modified)
        const unsigned long long inSlot = __ballot(st.fNode == entry && st.fKey != kE);
        if (inSlot) {
          if (st.fNode == entry && st.fKey != kE) st.fKey = key;
        } else {
          const int at = bag.find(entry);
          if (at < 0) return kAstarGrowHeap;   // cannot happen: an open node is in a slot or in the set
          bag.modify(entry, key);
          if (at == st.bmPos) { st.bmKey = key; st.bmCount = 1; }
          else if (key < st.bmKey) { st.bmKey = key; st.bmPos = at; st.bmNode = entry; st.bmCount = 1; }
          else if (key == st.bmKey) st.bmCount++;
        }
      } else {
        bag_push(key, entry);
      }
    }
  }
}

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
  AstarState st;
  const AEdge* edges = nav.aedges + (size_t)(uint32_t)uniform_i((int)s.poly_base) * kNvp;
#ifdef BPSX_PHASE_TIMING
#define ASTAR_RUN(M) astar_loop<M>(g, st, edges, endIp, endPos, pops, phase_acc, phase_t0)
#else
#define ASTAR_RUN(M) astar_loop<M>(g, st, edges, endIp, endPos, pops)
#endif
  float startTotal;
  auto begin = [&]() {
    g.clear();
    const float dx = endPos[0] - startPos[0], dy = endPos[1] - startPos[1], dz = endPos[2] - startPos[2];
    const float total = sqrtf(dx * dx + dy * dy + dz * dz) * 0.999f;
    g.nodeCount = 1;
    if (lane == 0) {
      GeoLds* L = g.L;
      ANode& hn = g.ws->nodes[0];
      for (int k = 0; k < 3; ++k) { L->w_pos[k][0] = startPos[k]; hn.pos[k] = startPos[k]; }
      L->w_cost[0] = 0; L->w_total[0] = total;
      hn.cost = 0; hn.total = total;
      hn.parent = 0;
      L->w_parent[0] = 0;
      L->n_link[0] = make_link(startIp, 1u, kChainEnd);   // open
      L->first[GeoWave::hash(startIp)] = 0;
    }
    wave_sync();
    st.lastBest = 0;
    st.lastBestCost = total;
    st.outOfNodes = false;
    startTotal = total;
  };
  AstarExit ex;
#if BPSX_BAG
  begin();
  st.bag.init();
  st.rh.init();
  if (lane == 0) g.ws->oplog[0] = OpLogEntry{__float_as_uint(startTotal), (startIp << 11) | (kOpPush << 30)};
  st.logPos = 1;
  st.logDone = 0;
  st.bmCount = 0; st.bmPos = 0; st.bmKey = OpenBag::kEmpty; st.bmNode = OpenBag::kNoNode;
  st.forceNode = OpenBag::kNoNode;
  // the start node waits in slot 0
  st.fKey = (lane >> 3) == 0 ? __float_as_uint(startTotal) : OpenBag::kEmpty;
  st.fNode = (lane >> 3) == 0 ? startIp << 11 : OpenBag::kNoNode;
  st.fe = AEdge{{0.f, 0.f, 0.f}, kNoNb};
  if (lane < kNvp) st.fe = edges[startIp * kNvp + (uint32_t)lane];
#ifdef BPSX_PHASE_TIMING
#define ASTAR_SPEC(S) astar_spec<S>(g, st, edges, endIp, endPos, pops, phase_acc, phase_t0)
#else
#define ASTAR_SPEC(S) astar_spec<S>(g, st, edges, endIp, endPos, pops)
#endif
  ex = ASTAR_SPEC(false);
  if (ex == kAstarGrowLinks) { g.linkSpills++; ex = ASTAR_SPEC(true); }
#undef ASTAR_SPEC
#else
  ex = kAstarGrowHeap;
#endif
  if (ex == kAstarGrowHeap) {
    // the open list has outgrown the register set (or the log its space): the search is done
    // again with the heap itself, which can spill
    if (BPSX_BAG) g.tieRestarts++;
    begin();
    st.rh.init();
    st.rh.push(__float_as_uint(startTotal), startIp << 11, lane);
    ex = ASTAR_RUN(0);
    if (ex == kAstarGrowLinks) { g.linkSpills++; ex = ASTAR_RUN(1); }
  }
  if (ex == kAstarGrowHeap) {
    g.heapSpills++;
    // the open list leaves the registers: entry q goes to index q - 1 of the LDS heap
    const RegHeap& rh = st.rh;
    auto put = [&](int i, uint32_t t, uint32_t n) {
      const HeapEntry e{__uint_as_float(t), n & 0x7ffu};
      if (i < kHeapLds) g.L->heap[i] = e;
      else { BPSX_KEEP_APART(); g.ws->heap_spill[i] = e; BPSX_KEEP_APART(); }
    };
    if (lane >= 1 && lane <= rh.size) put(lane - 1, rh.t0, rh.n0);
    if (64 + lane <= rh.size) put(63 + lane, rh.t1, rh.n1);
    g.heapSize = rh.size;
    wave_sync();
    ex = ASTAR_RUN(2);
  }
#undef ASTAR_RUN
  (void)ex;
  if (st.outOfNodes) return 0;   // no path to build: the result is a failure
  const int lastBest = st.lastBest;
  // getPathToNode: one walk up the parents notes the node indices (in the window's array of
  // positions, no longer needed), then all lanes fill the corridor, which overlays the hash heads;
  // the links stay readable while it is written
  static_assert(sizeof(g.L->w_pos) >= kMaxPath * sizeof(uint16_t), "the walk must fit the array it reuses");
  uint16_t* walk = reinterpret_cast<uint16_t*>(g.L->w_pos);
  wave_sync();
  int length = 0;
  for (int c = lastBest + 1; c && length <= kMaxNodes; c = uniform_i((int)g.ws->nodes[c - 1].parent)) {
    if (lane == 0 && length < kMaxPath) walk[length] = (uint16_t)(c - 1);
    length++;
  }
  wave_sync();
  const bool ok = length <= kMaxPath && link_id(g.link<true>(lastBest)) == endIp && !st.outOfNodes;
  if (!ok) return 0;
  for (int i = lane; i < length; i += 64) F->corridor[length - 1 - i] = (uint16_t)link_id(g.link<true>((int)walk[i]));
  wave_sync();
  return length;
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
  FunnelLds* F = &reinterpret_cast<GeoShared*>(g.L)->f;
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

}  // namespace BPSX_GEO_NS
}  // namespace bpsx
