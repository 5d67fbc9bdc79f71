// Geodesic distance on the GPU: Detour's A* over the polygon graph followed by the funnel
// (string pulling) and the summed segment length, with the exact buffer limits and failure
// conventions of the reference, so that the value equals PathFinder::findPath's.
//
// Execution model: one wavefront (64 lanes) owns one query at a time and pulls the next from
// a shared queue when done.  The search touches almost only nodes it created recently (the
// frontier of A* is narrow), so LDS holds what is hot and small and HBM holds the rest:
//   - the open list in registers: sorted by total, up to 256 entries (OpenList), which lets a
//     pass expand up to kRows nodes at once (astar_fast); the reference's binary heap, also in
//     registers while it has fewer than 128 entries (RegHeap, entry q in lane q mod 64), is
//     what a search falls back to when totals tie or the list outgrows its registers; a heap
//     longer than that (rare) keeps its top kHeapLds entries in LDS,
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
// BPSX_WINDOW, BPSX_HASH, BPSX_TAG_SLOTS), and everything that depends on them lives in namespace
// bpsx::BPSX_GEO_NS (default geo): the file can be included again with other values and
// another namespace name to get a second instantiation of the same search.
#include "nav_device.h"

#ifndef BPSX_GEODESIC_COMMON_H
#define BPSX_GEODESIC_COMMON_H
namespace bpsx {

#ifdef BPSX_PHASE_TIMING
// diagnostic build: cycles per phase of the sorted-list loop -> counters: 0 front of the list, 1 fetch, 2 lookup,
// 3 costs, 4 rows that stand, 5 closing, new nodes and stores, 6 list and log; 7 counts the passes
// (the comment that the asm statement leaves in the compiler's assembly output names the loop's
// instantiation and the mark, for tests/measure_astar_loop_phases.py)
#define FM(k) do { constexpr int slot_[11] = {7, 0, 1, 2, 3, 4, 5, 5, 5, 6, 6}; const unsigned long long now_ = __builtin_readcyclecounter(); \
    asm volatile("; astar_fast spill=%0 pairs=%1 mark=%2" :: "i"((int)S), "i"(P), "i"(k)); \
    if ((k) == 0) g.phase[7]++; else g.phase[slot_[k]] += now_ - g.phase_t0; g.phase_t0 = now_; } while (0)
#else
#define FM(k) do { } while (0)
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
// mask of the lanes where b holds (takes the condition as such, not widened to an integer and compared again)
BPSX_DEV unsigned long long lanes_where(bool b) { return __builtin_amdgcn_ballot_w64(b); }
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

// index of the lowest set bit, -1 for an empty mask (the instruction's own convention)
BPSX_DEV int first_lane(unsigned long long mask) {
  int r;
  asm("s_ff1_i32_b64 %0, %1" : "=s"(r) : "s"(mask));
  return r;
}
BPSX_DEV unsigned long long without_lane(unsigned long long mask, int lane) {
  asm("s_bitset0_b64 %0, %1" : "+s"(mask) : "s"(lane));
  return mask;
}
// a and b with lane `lane` replaced by va and vb (all three uniform): one M0 write for both
BPSX_DEV void wlane2(uint32_t& a, uint32_t va, uint32_t& b, uint32_t vb, int lane) {
  const int sa = __builtin_amdgcn_readfirstlane((int)va), sb = __builtin_amdgcn_readfirstlane((int)vb), sl = __builtin_amdgcn_readfirstlane(lane);
  asm("s_mov_b32 m0, %4\n\tv_writelane_b32 %0, %2, m0\n\tv_writelane_b32 %1, %3, m0" : "+v"(a), "+v"(b) : "s"(sa), "s"(sb), "s"(sl) : "m0");
}

// lanes 8..15 of each row of 16 take src of the lane 8 below them, lanes 0..7 keep low
// min(v, v of the lane that the DPP control names); lanes without such a lane, or outside the
// row mask (one bit per 16 lanes), keep v.  (The other lane's value defaults to the identity of
// the minimum, which lets the compiler fold the lane move into the v_min itself.)
template <int Ctrl, int RowMask> BPSX_DEV uint32_t umin_dpp(uint32_t v) {
  const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(-1, (int)v, Ctrl, RowMask, 0xf, false);
  return o < v ? o : v;
}
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
  if (__builtin_expect(lanes_where(xb - 1u < 0x0f800000u - 1u) != 0, 0)) return sqrtf(x);   // 0 < x < 2^-96 in some lane: never in practice
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
  // constants of the lane: the positions that must each be the smaller of their sibling pair
  // for the hole of a pop to pass through position `lane` (itself and its ancestors below the
  // root), as a bit set, and the same for the parent of position 64 + lane
  uint32_t anc0, anc1, panc0, panc1;
  static constexpr uint32_t kEmpty = 0x7fffffffu;   // above +inf; every key stays below 2^31
  static BPSX_DEV unsigned long long route_set(int q) {
    unsigned long long m = 0;
    for (; q >= 2; q >>= 1) m |= 1ull << q;
    return m;
  }
  BPSX_DEV void init(int lane) {
    t0 = t1 = kEmpty; n0 = n1 = 0; size = 0;
    const unsigned long long a = route_set(lane), pa = route_set(32 + (lane >> 1));
    anc0 = (uint32_t)a; anc1 = (uint32_t)(a >> 32);
    panc0 = (uint32_t)pa; panc1 = (uint32_t)(pa >> 32);
  }
  // v of the neighbouring lane (lane ^ 1)
  static BPSX_DEV uint32_t quad_swap(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xb1 /* quad_perm:[1,0,3,2] */, 0xf, 0xf, false);
  }
  static BPSX_DEV uint32_t xlane(int src_lane, uint32_t v) {   // v of another lane; all lanes must be active
    return (uint32_t)__builtin_amdgcn_ds_bpermute(src_lane * 4, (int)v);
  }

  // dtNodeQueue::bubbleUp of entry (t, n) from position q, by all lanes at once.  The lanes on
  // the way from q to the root read their parent's entry; ancestors with a greater key move
  // one step down that way (they form a run from q upwards: keys never increase towards the
  // root) and the entry lands on top of the run.  Positions 64..127 have all their ancestors
  // in the first pair, so only q itself can be in the second.
  template <bool W = true> BPSX_DEV void bubble_up(int q, uint32_t t, uint32_t n, int lane) {
    const int up = (31 - __clz(q)) - (31 - __clz(lane));   // lane 0 (clz 32) is no heap position
    const bool on = lane >= 1 && up >= 0 && (q >> (up & 31)) == lane;
    const uint32_t pk = xlane(lane >> 1, t0), pn = xlane(lane >> 1, n0);
    const bool parentMoves = on && lane > 1 && pk > t;
    const bool vacant = lane == q || t0 > t;
    const bool land = on && vacant && !parentMoves;
    if (W && q >= 64) {
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
  // heap position of node n's entry, 0 if it has none
  template <bool W = true> BPSX_DEV int position(uint32_t n, int lane) const {
    const unsigned long long m0 = lanes_where(lane >= 1 && lane <= size && n0 == n);
    if (m0) return __ffsll((long long)m0) - 1;
    if (!W || size < 64) return 0;
    const unsigned long long m1 = lanes_where(64 + lane <= size && n1 == n);
    return m1 ? 64 + __ffsll((long long)m1) - 1 : 0;
  }
  // push (open false) or modify (open true) through one copy of the walk; an open node without
  // an entry (there is none) would be a walk from position 0, which changes nothing
  // Most entries stay where they start (a new total is rarely below its parent's): that case is
  // two lane writes on the scalar unit's word, without the lane-parallel walk.
  template <bool W = true> BPSX_DEV void update(bool open, uint32_t n, uint32_t t, int lane) {
    int q;
    if (open) q = position<W>(n, lane);
    else q = ++size;
    const uint32_t pk = rlane(t0, q >> 1);   // position 0 holds kEmpty: no entry (q = 0) and the root take the walk
    if (pk <= t) {
      if (!W || q < 64) { t0 = wlane(t0, t, q); n0 = wlane(n0, n, q); }
      else { t1 = wlane(t1, t, q & 63); n1 = wlane(n1, n, q & 63); }
      return;
    }
    bubble_up<W>(q, t, n, lane);
  }
  // dtNodeQueue::pop after the caller has taken the root.  The reference moves the hole left
  // by the root down to a leaf along the smaller children and then bubbles the former last
  // entry up from there; along that route keys never decrease, so the entry ends up above the
  // first route element greater than it and nothing below moves.  Which child the hole moves to
  // depends only on the children's keys, which the moves above them do not change, so the
  // route is known at once: siblings sit in neighbouring lanes, one comparison with the
  // neighbour says for every position whether it is the smaller of its pair (the left one when
  // equal), and a position is on the route when that holds for itself and all its ancestors,
  // a test of the ballot against a per-lane constant.  Then every route position whose
  // smaller child is not greater than the entry takes that child, and the first one whose
  // child is greater takes the entry.  Positions past the end hold kEmpty and never move.
  // W false: the caller knows that the list has fewer than 64 entries.
  template <bool W = true> BPSX_DEV void pop(int lane) {
    const int last = size;
    size--;
    uint32_t lt, ln;
    if (!W || last < 64) { lt = rlane(t0, last); ln = rlane(n0, last); t0 = wlane(t0, kEmpty, last); }
    else { lt = rlane(t1, last & 63); ln = rlane(n1, last & 63); t1 = wlane(t1, kEmpty, last & 63); }
    if (size == 0) return;
    const bool wide = W && size >= 64;      // entries in the second pair
    const bool lo = lane < 32;              // children of positions 32..63 are in the second pair
    constexpr unsigned long long kOdd = 0xaaaaaaaaaaaaaaaaull;
    // less0: the position's key is below its sibling's.  A right child is the smaller one when
    // that holds, a left child unless it holds for its right neighbour.
    const unsigned long long less0 = lanes_where(t0 < quad_swap(t0));
    const unsigned long long lose0 = ~((less0 & kOdd) | (~(less0 >> 1) & ~kOdd));
    unsigned long long less1 = 0;
    if (wide) less1 = lanes_where(t1 < quad_swap(t1));
    const bool on = lane >= 1 && ((anc0 & (uint32_t)lose0) | (anc1 & (uint32_t)(lose0 >> 32))) == 0;
    // the smaller child of this lane's position: the right one if its key is below the left one's
    const int c0 = (2 * lane) & 63;
    const unsigned long long lessc = lo ? less0 : less1;
    const int c = c0 + (int)((uint32_t)(lessc >> (c0 + 1)) & 1u);
    uint32_t ck = xlane(c, t0), cn = xlane(c, n0);
    if (wide) {
      const uint32_t hk = xlane(c, t1), hn = xlane(c, n1);
      ck = lo ? ck : hk; cn = lo ? cn : hn;
    } else {
      ck = lo ? ck : kEmpty;
    }
    const bool take = on && ck <= lt;
    const bool land = on && !take && (lane == 1 || t0 <= lt);
    if (wide) {
      // positions 64..127 have no children: the one on the route takes the entry if its parent took it
      const unsigned long long lose1 = ~((less1 & kOdd) | (~(less1 >> 1) & ~kOdd));
      const bool here = ((lose1 >> lane) & 1ull) == 0 && ((panc0 & (uint32_t)lose0) | (panc1 & (uint32_t)(lose0 >> 32))) == 0 && t1 <= lt;
      t1 = here ? lt : t1;
      n1 = here ? ln : n1;
    }
    t0 = take ? ck : (land ? lt : t0);
    n0 = take ? cn : (land ? ln : n0);
  }
};

// The open list as a sorted array in registers.  dtNodeQueue::pop returns the entry with the
// smallest total; while that smallest total is held by one entry only, which entry that is
// does not depend on how the reference's binary heap happens to be arranged.  So a search can
// keep its open list in any form that yields the minimum, as long as it notices when two
// entries share the smallest total (a tie, about one pop in ten thousand) and then asks the
// exact heap.  Sorted by total, entry i in lane i & 63 of pair i >> 6: the next nodes to expand
// are the first lanes, a pop is a shift of all lanes by one, and an insertion is one comparison
// of all lanes with the new total and a shift of those above it.  Unused places hold kEmpty
// keys and kNone nodes.  Entries with equal totals sit next to each other in no defined order.
struct OpenList {
  static constexpr int kPairs = 4;
  uint32_t t[kPairs], n[kPairs];   // totals as bit patterns (see RegHeap), nodes packed like RegHeap's
  int size;
  static constexpr uint32_t kEmpty = 0x7fffffffu;
  static constexpr uint32_t kNone = 0xffffffffu;    // no packed node looks like this (26 bits)
  BPSX_DEV void init() { t[0] = kEmpty; n[0] = kNone; size = 0; }   // further pairs are cleared when the list grows into them
  BPSX_DEV void clear_pair(int k) { t[k] = kEmpty; n[k] = kNone; }
  // lane L takes v of lane L - 1, lane 0 keeps `first`
  static BPSX_DEV uint32_t up1(uint32_t first, uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)first, (int)v, 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
  }
  // lane L takes v of lane L + 1, lane 63 keeps `last`
  static BPSX_DEV uint32_t down1(uint32_t last, uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)last, (int)v, 0x130 /* wave_shl:1 */, 0xf, 0xf, false);
  }
  // v as a select operand under a lane mask held in scalar registers
  static BPSX_DEV uint32_t pick(unsigned long long mask, uint32_t yes, uint32_t no) {
    uint32_t r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(no), "v"(yes), "s"(mask));
    return r;
  }
  // The first c entries leave.  P: register pairs in use (64 entries each).
  template <int P> BPSX_DEV void drop_front(int c, int lane) {
    if (P == 1) {
      for (int i = 0; i < c; ++i) { t[0] = down1(kEmpty, t[0]); n[0] = down1(kNone, n[0]); }
    } else {
      const int src = ((lane + c) & 63) * 4;
      uint32_t a[P], b[P];
#pragma unroll
      for (int k = 0; k < P; ++k) { a[k] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)t[k]); b[k] = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)n[k]); }
      const bool same = lane + c < 64;
#pragma unroll
      for (int k = 0; k < P; ++k) {
        t[k] = same ? a[k] : (k + 1 < P ? a[k + 1 < P ? k + 1 : k] : kEmpty);
        n[k] = same ? b[k] : (k + 1 < P ? b[k + 1 < P ? k + 1 : k] : kNone);
      }
    }
  }
  // the number of entries, after drops and updates (which do not keep it)
  template <int P> BPSX_DEV void count() {
    size = 0;
#pragma unroll
    for (int k = 0; k < P; ++k) size += __popcll(lanes_where(t[k] != kEmpty));
  }
  // lane L takes v of lane L - 1 (lane 0: anything)
  static BPSX_DEV uint32_t from_below(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x138 /* wave_shr:1 */, 0xf, 0xf, true);
  }
  // Node n_ gets total t_: its entry, if it has one, leaves, and the new entry goes behind those
  // with totals up to t_.  (A node has an entry exactly when it is open and has not just been
  // taken off the front, so whether this is the reference's push or its modify need not be told.)
  template <int P> BPSX_DEV void update(uint32_t n_, uint32_t t_, int lane) {
    if (P == 1) {
      // No branches: without an old entry its place is -1, as an unsigned bound that keeps every lane
      const unsigned long long g0 = lanes_where(t[0] > t_), h0 = lanes_where(n[0] == n_);
      const unsigned long long m0 = g0 & (h0 | (h0 - 1ull));   // the lanes up to the old entry's; without one, all
      const int p = first_lane(m0);   // never empty: the unused places compare greater
      t[0] = pick(m0, from_below(t[0]), t[0]);
      n[0] = pick(m0, from_below(n[0]), n[0]);
      wlane2(t[0], t_, n[0], n_, p);
      return;
    }
    unsigned long long m[P];
    int rp = -1, rl = 0;   // pair and lane of the old entry
#pragma unroll
    for (int k = 0; k < P; ++k) {
      m[k] = lanes_where(t[k] > t_);
      const unsigned long long h = lanes_where(n[k] == n_);
      if (h && rp < 0) { rp = k; rl = __ffsll((long long)h) - 1; }
    }
    // only the entries from the new place up to the old one move
    int pp = -1, pl = 0;   // pair and lane of the new place
#pragma unroll
    for (int k = 0; k < P; ++k) {
      if (rp >= 0 && k > rp) m[k] = 0;
      if (k == rp) m[k] &= (2ull << rl) - 1ull;
      if (m[k] && pp < 0) { pp = k; pl = __ffsll((long long)m[k]) - 1; }
    }
#pragma unroll
    for (int k = P - 1; k >= 1; --k) {
      const uint32_t ct = rlane(t[k - 1], 63), cn = rlane(n[k - 1], 63);   // what moves up into pair k
      t[k] = pick(m[k], up1(ct, t[k]), t[k]);
      n[k] = pick(m[k], up1(cn, n[k]), n[k]);
    }
    t[0] = pick(m[0], from_below(t[0]), t[0]);
    n[0] = pick(m[0], from_below(n[0]), n[0]);
#pragma unroll
    for (int k = 0; k < P; ++k)
      if (pp == k) wlane2(t[k], t_, n[k], n_, pl);
  }
};

struct AstarState {
  int lastBest;      // the goal's node once it has been popped
  bool outOfNodes;
  RegHeap rh;        // the reference's heap: always (exact loops), or as of log record `synced` (sorted-list loop)
  OpenList ol;
  int logEnd;        // records in the slot's operation log
  int synced;        // records already applied to rh
};

// Applies log records [st.synced, st.logEnd) to the reference's heap, pass by pass.  Records are
// fetched 64 at a time, one per lane, and again when the next pass is not among them in full
// (a pass has at most 1 + 8 * 6 records).  False when the heap
// outgrows the registers.
BPSX_DEV bool replay_log(const OpRec* log, AstarState& st, int lane) {
  RegHeap& rh = st.rh;
  int base = -64;              // record held by lane 0
  uint32_t rk = 0, rw = 0;
  auto fetch = [&](int from) {
    base = from;
    rk = 0; rw = 0;
    if (base + lane < st.logEnd) { const OpRec r = log[base + lane]; rk = r.key; rw = r.word; }
  };
  for (int pos = st.synced; pos < st.logEnd;) {
    // a fetch is a round trip to HBM: one only when the pass at hand is not all there
    if (pos >= base + 64) fetch(pos);
    if (pos - base + 1 + (int)(rlane(rk, pos - base) >> 8) > 64) fetch(pos);
    const int h = pos - base;
    const uint32_t hk = rlane(rk, h), hw = rlane(rw, h);
    const int c = (int)(hk & 0xffu), nrec = (int)(hk >> 8);
    // rows in the reference's order: the first two swap when the heap has row 1's node on top
    const bool swap = (hw & kOpUnordered) && rlane(rh.n0, 1) != (hw & 0x3ffffffu);
    const bool mine = lane > h && lane <= h + nrec;
    const int myRow = (int)((rw >> 26) & 7u);
    for (int i = 0; i < c; ++i) {
      const int row = (swap && i < 2) ? 1 - i : i;
      rh.pop(lane);
      unsigned long long m = lanes_where(mine && myRow == row);
      while (m) {
        const int j = __ffsll((long long)m) - 1;
        m &= m - 1;
        const uint32_t key = rlane(rk, j), word = rlane(rw, j);
        const uint32_t node = word & 0x3ffffffu;
        // a node seen as open whose entry has left (its row came earlier in the pass) is pushed
        int q = ((word >> 29) & 1u) ? rh.position(node, lane) : 0;
        if (!q) {
          if (rh.size >= kRegHeap) return false;
          q = ++rh.size;
        }
        rh.bubble_up(q, key, node, lane);
      }
    }
    pos += 1 + nrec;
  }
  st.synced = st.logEnd;
  return true;
}
enum AstarExit { kAstarEmpty = 0, kAstarGoal = 1, kAstarGrowLinks = 2, kAstarGrowHeap = 3, kAstarTie = 4, kAstarLogFull = 5 };

// Two roots at once: one test of the arguments' range for both.
BPSX_DEV void sqrt_exact2(float x, float y, float* rx, float* ry) {
  const uint32_t xb = __float_as_uint(x), yb = __float_as_uint(y);
  if (__builtin_expect(lanes_where(xb - 1u < 0x0f800000u - 1u || yb - 1u < 0x0f800000u - 1u) != 0, 0)) {
    *rx = sqrtf(x); *ry = sqrtf(y);   // 0 < argument < 2^-96 in some lane: never in practice
    return;
  }
  const float s = __builtin_amdgcn_sqrtf(x), t = __builtin_amdgcn_sqrtf(y);
  const float sd = __uint_as_float(__float_as_uint(s) - 1u), su = __uint_as_float(__float_as_uint(s) + 1u);
  const float td = __uint_as_float(__float_as_uint(t) - 1u), tu = __uint_as_float(__float_as_uint(t) + 1u);
  float r = fmaf(-sd, s, x) <= 0.0f ? sd : s;
  r = fmaf(-su, s, x) > 0.0f ? su : r;
  float q = fmaf(-td, t, y) <= 0.0f ? td : t;
  q = fmaf(-tu, t, y) > 0.0f ? tu : q;
  *rx = r; *ry = q;
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
#define BPSX_LINKS_LDS 1016
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
#ifndef BPSX_TAG_SLOTS
#define BPSX_TAG_SLOTS 256
#endif
constexpr int kTagSlots = BPSX_TAG_SLOTS;
constexpr int kRows = 8;                    // nodes expanded per pass of astar_fast, one per row of 64 / kRows lanes
constexpr int kRowLanes = 64 / kRows;
constexpr int kRowShift = 3;
static_assert(kRowLanes == (1 << kRowShift) && kRowLanes > kNvp, "a row needs a lane per edge and one for the node itself");
// lanes of the rows below j
constexpr unsigned long long rows_below(int j) { return j * kRowLanes >= 64 ? ~0ull : (1ull << (j * kRowLanes)) - 1ull; }
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
  uint32_t tag[kTagSlots];         // which nodes of a pass touch a polygon (see astar_fast)
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
  uint32_t tagNow;                   // mark of the current pass in L->tag, counting down
#ifdef BPSX_PHASE_TIMING
  unsigned long long phase[8], phase_t0;
#endif
  uint32_t exactRuns;                // queries run again with the exact heap
  uint32_t tieReplays;               // ties resolved by replaying the operation log through the exact heap
  uint32_t pairTies;                 // passes that took two nodes of equal total in one go

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
  // the multiply as the full-rate 24-bit instruction (polygon indices have 15 bits)
  static BPSX_DEV uint32_t hash(uint32_t ip) {
    uint32_t m;
    asm("v_mul_u32_u24 %0, %1, %2" : "=v"(m) : "v"(ip), "s"(0x9e3779u));
    return (m >> 9) & (kHashSize - 1);
  }
  BPSX_DEV void clear() {
    for (int i = lane; i < kHashSize; i += 64) L->first[i] = (uint16_t)kChainEnd;
    for (int i = lane; i < kTagSlots; i += 64) L->tag[i] = 0xffffffffu;
    tagNow = 0x1fffffffu;
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
    while (lanes_where(cur != kChainEnd)) {
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
      const unsigned long long m = lanes_where(i < heapSize && (int)hget<S>(i).node == n);
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

// The expansion loop of findPath for an open list that has left the registers (more than
// kRegHeap entries: an obstacle-free hall does it, the benchmark's mazes and rooms do not): the
// reference's heap in LDS/HBM, one node per pass, links wherever they are.
BPSX_DEV AstarExit astar_loop(GeoWave& g, AstarState& st, const AEdge* edges, uint32_t endIp, const float* endPos, uint32_t* pops) {
  const int lane = g.lane;
  GeoLds* L = g.L;
  const float H_SCALE = 0.999f;
  const float e0 = endPos[0], e1 = endPos[1], e2 = endPos[2];
  endIp = (uint32_t)uniform_i((int)endIp);   // the same in all lanes: the goal test stays on the scalar unit
  constexpr bool S = true;    // links and states may be in HBM
  while (g.heapSize > 0) {
    // the node about to be popped is the root: fetch its edges while the heap is repaired
    const int bi = uniform_i((int)L->heap[0].node);
    const uint32_t blink = g.link<S>(bi);   // the node's link word: closing the node rewrites its flags
    const uint32_t bestIp = link_id((uint32_t)uniform_i((int)blink));
    uint32_t nb = kNoNb;
    float m0 = 0, m1 = 0, m2 = 0;
    if (lane < kNvp) {
      const AEdge e = edges[bestIp * kEdgeStride + lane];
      nb = e.nb; m0 = e.mid[0]; m1 = e.mid[1]; m2 = e.mid[2];
    }
    float b0, b1, b2, bcost;
    uint32_t bparent;   // read now, moved to a scalar register only after the pop
    if (g.in_window(bi)) {
      const int w = bi & (kWindow - 1);
      b0 = L->w_pos[0][w]; b1 = L->w_pos[1][w]; b2 = L->w_pos[2][w]; bcost = L->w_cost[w];
      BPSX_KEEP_APART(); bparent = g.ws->nodes[bi].parent; BPSX_KEEP_APART();   // the heap lies over the window's parent indices
    } else {
      BPSX_KEEP_APART();
      const float4 pc = *reinterpret_cast<const float4*>(g.ws->nodes[bi].pos);   // pos, cost
      b0 = pc.x; b1 = pc.y; b2 = pc.z; bcost = pc.w;
      bparent = g.ws->nodes[bi].parent;
      BPSX_KEEP_APART();
    }
    g.pop<S>();
    const uint32_t pidx = (uint32_t)uniform_i((int)bparent);
    g.set_link<S>(bi, with_flags(blink, 2u));   // open -> closed
    if (bestIp == endIp) { st.lastBest = bi; return kAstarGoal; }
    (*pops)++;
    const uint32_t bucket = GeoWave::hash(nb);
    uint32_t chainHead, hitLink;
    int ni = g.find<S>(nb != kNoNb, nb, bucket, &chainHead, &hitLink);
    // the polygon the expanded node was reached from is not entered again
    if (pidx && ni + 1 == (int)pidx) nb = kNoNb;
    // new nodes take consecutive indices in edge order
    const bool isNew = nb != kNoNb && ni < 0;
    const unsigned long long need = lanes_where(isNew);
    if (need) {
      const int rank = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(need >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)need, 0u));
      const int count = __popcll(need);
      const int want = g.nodeCount + count;
      // the reference carries on without the nodes that do not fit, but reports anything found
      // after that as failure (only plain DT_SUCCESS counts, PathFinder.cpp:506): the search can stop
      if (want > kMaxNodes) { st.outOfNodes = true; return kAstarEmpty; }
      if (isNew) ni = g.nodeCount + rank;
      g.nodeCount = want;
      bool pending = isNew;
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
        if (!lanes_where(pending)) break;
      }
    }
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
    if (lanes_where(miss)) {
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
      }
      *reinterpret_cast<float4*>(hn.pos) = make_float4(p0, p1, p2, cost);
      *reinterpret_cast<uint2*>(&hn.total) = make_uint2(__float_as_uint(total), (uint32_t)(bi + 1));   // total, parent = expanded node
      g.ws->parents[ni] = (uint16_t)(bi + 1);
    }
    wave_sync();
    // ---- ordered phase, in edge order: the open list.  (findPath's "nearest so far" record,
    // lastBestNode, is not kept: it only matters to a search that ends without reaching the
    // goal, and the caller reports DT_PARTIAL_RESULT as failure, PathFinder.cpp:506.)
    unsigned long long upd = lanes_where(update);
    const unsigned long long openMask = lanes_where(wasOpen);
    while (upd) {
      const int src = __ffsll((long long)upd) - 1;
      upd &= upd - 1;
      const int node = (int)rlane((uint32_t)ni, src);
      const float t = lane_f(total, src);
      if ((openMask >> src) & 1ull) g.modify<S>(node, t);
      else g.push<S>(t, node);
    }
  }
  return kAstarEmpty;
}

// The same loop for an open list in registers (S as above), two nodes per pass.  Besides the
// node at the root (A, lanes 0..5) the pass works on the smaller child of the root (B, lanes
// 16..21), which is what the reference pops next unless A's expansion puts something smaller
// on the list: the edge records of both arrive in one load, and node lookup, costs, node
// creation and stores of both are done by the same instructions.  B's results are computed
// from the state before A's expansion; they are what the reference computes after it when
//   - every total A puts on the open list is at least B's (B stays at the root: an entry
//     moves past its parent only when its key is smaller),
//   - A created or updated no node that B read (a neighbour of both) and not B's own node
//     (A's own node is closed before either looks anything up, as it is when B's turn comes),
// and B is not the goal.  Then the pass applies A's and B's updates in the reference's order:
// new nodes take consecutive indices, A's first; the "nearest so far" record and the open
// list see A's updates in edge order, then B's pop, then B's updates.  Otherwise B's lanes
// are dropped and B becomes A of the next pass.
template <bool S, bool W>
BPSX_DEV AstarExit astar_loop2(GeoWave& g, AstarState& st, const AEdge* edges, uint32_t endIp, const float* endPos, uint32_t* pops) {
  const int lane = g.lane;
  GeoLds* L = g.L;
  const float H_SCALE = 0.999f;
  const float e0 = endPos[0], e1 = endPos[1], e2 = endPos[2];
  endIp = (uint32_t)uniform_i((int)endIp);
  RegHeap& rh = st.rh;
  const bool rowB = lane >= 16;
  const int el = lane & 15;                      // edge handled by this lane
  const bool edgeLane = el < kNvp && lane < 32;
  while (rh.size > 0) {
    if (!S && g.nodeCount > kLinksLds - 2 * kNvp) return kAstarGrowLinks;
    if (rh.size > (W ? kRegHeap : 63) - 2 * kNvp) return kAstarGrowHeap;   // W false: all entries in the first register pair
    const uint32_t rootA = rlane(rh.n0, 1);
    const int biA = (int)(rootA & 0x7ffu);
    const uint32_t ipA = rootA >> 11;
    const uint32_t kl = rlane(rh.t0, 2), kr = rlane(rh.t0, 3);   // kEmpty past the end
    const uint32_t nl = rlane(rh.n0, 2), nr = rlane(rh.n0, 3);
    const uint32_t rootB = kr < kl ? nr : nl;
    const uint32_t keyB = kr < kl ? kr : kl;
    const int biB = (int)(rootB & 0x7ffu);
    const uint32_t ipB = rootB >> 11;
    const bool spec = rh.size >= 2 && ipA != endIp && ipB != endIp;
    const uint32_t blinkA = g.link<S>(biA);
    const uint32_t blinkB = g.link<S>(spec ? biB : biA);   // unchanged by A whenever B is committed
    const bool act = edgeLane && (!rowB || spec);
    const int bi = (rowB && spec) ? biB : biA;   // the node this lane expands
    uint32_t nb = kNoNb;
    float m0 = 0, m1 = 0, m2 = 0;
    if (act) {
      const AEdge e = edges[(rowB ? ipB : ipA) * kEdgeStride + (uint32_t)el];
      nb = e.nb; m0 = e.mid[0]; m1 = e.mid[1]; m2 = e.mid[2];
    }
    float b0, b1, b2, bcost;
    uint32_t bparent;
    {
      const int w = bi & (kWindow - 1);
      const bool binw = g.in_window(bi);
      b0 = L->w_pos[0][w]; b1 = L->w_pos[1][w]; b2 = L->w_pos[2][w]; bcost = L->w_cost[w];
      bparent = L->w_parent[w];
      if (lanes_where(!binw)) {
        if (!binw) {
          BPSX_KEEP_APART();
          const float4 pc = *reinterpret_cast<const float4*>(g.ws->nodes[bi].pos);   // pos, cost
          b0 = pc.x; b1 = pc.y; b2 = pc.z; bcost = pc.w;
          bparent = g.ws->nodes[bi].parent;
          BPSX_KEEP_APART();
        }
      }
    }
    rh.template pop<W>(lane);
    g.set_link<S>(biA, with_flags(blinkA, 2u));   // open -> closed
    if (ipA == endIp) { st.lastBest = biA; return kAstarGoal; }
    (*pops)++;
    const uint32_t bucket = GeoWave::hash(nb);
    uint32_t chainHead, hitLink;
    int ni = g.find<S>(nb != kNoNb, nb, bucket, &chainHead, &hitLink);
    // the polygon the expanded node was reached from is not entered again
    if (bparent && ni + 1 == (int)bparent) nb = kNoNb;
    // ---- costs of both nodes' steps (new nodes have no index yet and read slot 0)
    const bool isNew = nb != kNoNb && ni < 0;
    const bool valid = nb != kNoNb;
    const int nis = (valid && !isNew) ? ni : 0;
    const int rw = nis & (kWindow - 1);
    uint32_t fl = link_flags(hitLink);
    float p0 = L->w_pos[0][rw], p1 = L->w_pos[1][rw], p2 = L->w_pos[2][rw], oldTotal = L->w_total[rw];
    const bool miss = valid && !isNew && !g.in_window(nis);
    if (lanes_where(miss)) {
      if (miss) {
        const ANode& hn = g.ws->nodes[nis];
        BPSX_KEEP_APART();
        const float4 pc = *reinterpret_cast<const float4*>(hn.pos);     // pos, cost
        p0 = pc.x; p1 = pc.y; p2 = pc.z; oldTotal = hn.total;
        BPSX_KEEP_APART();
      }
    }
    if (isNew) { p0 = m0; p1 = m1; p2 = m2; fl = 0; }
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
    bool update = valid && !(fl && total >= oldTotal);
    // ---- does B stand?
    bool two = false;
    if (spec) {
      const uint32_t anb = (update && !rowB) ? nb : kNoNb;   // a lane of A that updates nothing leaves its node as B saw it
      const uint32_t bnb = (valid && rowB) ? nb : kNoNb - 1u;   // never equal to anb of an idle lane
      uint32_t clash = (uint32_t)(!rowB && update) & ((uint32_t)(__float_as_uint(total) < keyB) | (uint32_t)(nb == ipB));
#pragma unroll
      for (int j = 0; j < kNvp; ++j) clash |= (uint32_t)(bnb == rlane(anb, j));
      two = !lanes_where(clash != 0);
    }
    update = update & (!rowB | two);   // B's lanes are dropped unless B stands
    const bool wasOpen = update && (fl & 1u) != 0;
    // ---- new nodes take consecutive indices in edge order, A's before B's
    {
      const bool mine = isNew && update;   // a new node is always taken
      const unsigned long long need = lanes_where(mine);
      if (need) {
        const int rank = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(need >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)need, 0u));
        const int count = __popcll(need);
        const int want = g.nodeCount + count;
        // the reference carries on without the nodes that do not fit, but reports anything found
        // after that as failure (only plain DT_SUCCESS counts, PathFinder.cpp:506): stop
        if (S && want > kMaxNodes) { st.outOfNodes = true; return kAstarEmpty; }
        if (mine) ni = g.nodeCount + rank;
        g.nodeCount = want;
        // All insert at once in front of the chain head their lookup saw.  Of several that share a
        // bucket one store wins; the others see that when they read the head back and go round
        // again behind the winner.  One new node needs no check.
        bool pending = mine;
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
          if (!lanes_where(pending)) break;
        }
      }
    }
    if (update) {
      ANode& hn = g.ws->nodes[ni];
      const int w = ni & (kWindow - 1);
      const uint32_t parent = (uint32_t)bi + 1u;
      if (!isNew) g.set_link<S>(ni, with_flags(hitLink, 1u));   // open (again)
      if (g.in_window(ni)) {
        L->w_pos[0][w] = p0; L->w_pos[1][w] = p1; L->w_pos[2][w] = p2;
        L->w_cost[w] = cost; L->w_total[w] = total;
        L->w_parent[w] = (uint16_t)parent;
      }
      *reinterpret_cast<float4*>(hn.pos) = make_float4(p0, p1, p2, cost);
      *reinterpret_cast<uint2*>(&hn.total) = make_uint2(__float_as_uint(total), parent);
      g.ws->parents[ni] = (uint16_t)parent;
    }
    wave_sync();
    // ---- ordered phase, in the reference's order: A's lanes come before B's.  (findPath's
    // "nearest so far" record, lastBestNode, is not kept: it only matters to a search that ends
    // without reaching the goal, which the caller reports as failure, PathFinder.cpp:506.)
    const uint32_t packed = (uint32_t)ni | (nb << 11);
    const unsigned long long upd = lanes_where(update);
    const unsigned long long openMask = lanes_where(wasOpen);
    auto apply = [&](unsigned long long m) {
      while (m) {
        const int src = __ffsll((long long)m) - 1;
        m &= m - 1;
        rh.template update<W>((openMask >> src) & 1ull, rlane(packed, src), __float_as_uint(lane_f(total, src)), lane);
      }
    };
    apply(upd & 0xffffull);
    if (two) {   // A's updates are in: B leaves the open list
      rh.template pop<W>(lane);
      g.set_link<S>(biB, with_flags(blinkB, 2u));
      (*pops)++;
      apply(upd & ~0xffffull);
    }
  }
  return kAstarEmpty;
}

// The expansion loop with the open list as a sorted array (OpenList), up to kRows nodes per
// pass.  Row r of kRowLanes lanes works on entry r of the list (lane kRowLanes r + j on edge j
// of its polygon, the lane after the last edge on the node itself): the edge records of all of them arrive in one load, and node lookup, costs, node
// creation and stores are done by the same instructions for all rows.  Every row computes
// from the state before the pass.  Rows 0 .. c-1 are what the reference does next, in that
// order, when for every row j below c
//   - entry j's total is below entry j + 1's, and every total that an earlier row puts on the
//     open list is above it: entry j is then the only entry with the smallest total when its
//     turn comes, whatever the arrangement of the reference's heap,
//   - no earlier row creates or updates row j's own node or a node that row j updates too (a
//     neighbour of both).  A neighbour that row j reads and leaves alone, because the way
//     through row j is no better than the node's total, may be updated by an earlier row: its
//     total only gets lower.  This is found with one LDS word per polygon hash: every lane that
//     updates notes the pass and its row there (the earliest row wins), then these lanes and
//     the rows' own lanes look for a note of an earlier row.  Two polygons with the same hash
//     only make c smaller.
//   - entry j is not the goal (the goal ends the search when it is first in line).
// The pass commits c >= 1 rows: their new nodes take consecutive indices in row and edge
// order, their entries leave the list, their updates enter it.  A later row may improve the
// node of an earlier one (it sees it as open, the reference as closed): both views lead to
// the same node state and the same list, because a modify that finds no entry is a push.
// Returns kAstarTie when the first two entries share the smallest total.
template <bool S, int P>
BPSX_DEV AstarExit astar_fast(GeoWave& g, AstarState& st, const AEdge* edges, uint32_t endIp, const float* endPos, uint32_t* pops,
                             bool frontResolved) {
  const int lane = g.lane;
  GeoLds* L = g.L;
  const float H_SCALE = 0.999f;
  const float e0 = endPos[0], e1 = endPos[1], e2 = endPos[2];
  endIp = (uint32_t)uniform_i((int)endIp);
  OpenList& ol = st.ol;
  const int row = lane >> kRowShift, el = lane & (kRowLanes - 1);
  const bool edgeLane = el < kNvp;
  const bool ownLane = el == kNvp;   // looks after the row's own node in the conflict test
  constexpr unsigned long long kRowStart = 0x0101010101010101ull;   // the first lane of every row
  constexpr unsigned long long kRows1 = rows_below(1), kRows2 = rows_below(2);   // lanes of the first rows
  unsigned long long resolved = frontResolved ? 1ull : 0ull;
  // Written for few instructions on the common path: what is rare sits behind one branch each,
  // and conditions that feed a ballot are folded into the compared value first, so that the
  // ballot is the comparison's own result.
  for (;;) {
    if (ol.size <= 0) return kAstarEmpty;
    if (!S && g.nodeCount > kLinksLds - kRows * kNvp) return kAstarGrowLinks;
    if (st.logEnd > kOpLogCap - (1 + kRows * kNvp)) return kAstarLogFull;
    FM(0);
    // ---- how many entries at the front are each the only one with their total
    const unsigned long long uniq = lanes_where(ol.t[0] < OpenList::down1(OpenList::kEmpty, ol.t[0]));
    int lim = __builtin_ctzll(~uniq | (1ull << kRows));
    const uint32_t cand = (uint32_t)__builtin_amdgcn_ds_bpermute(row * 4, (int)ol.n[0]);   // entry `row`
    const int bi = (int)(cand & 0x7ffu);
    const uint32_t ip = cand >> 11;
    const unsigned long long goal = lanes_where(ip == endIp) & kRowStart;
    bool pairTie = false, goalInPair = false;
    if (__builtin_expect((goal | ((uniq & 1ull) ^ 1ull) | resolved) != 0, 0)) {
      if (resolved) { lim = 1; resolved = 0; }   // the caller has put the reference's next node first
      else if (lim == 0) {
        // The first two entries share the smallest total.  When they are alone in that and their
        // expansions are independent of each other (neither updates what the other reads, and
        // whatever they put on the list lies above their total), the reference expands them one
        // after the other, in the order its heap has them in, and ends in the same state either
        // way: the pass takes both and notes in the log that their order is open.
        if (!(uniq & 2ull)) return kAstarTie;
        pairTie = true;
        g.pairTies++;   // counts the attempts: one that fails comes back through the log
        lim = __builtin_ctzll(~(uniq | 3ull) | (1ull << kRows));
      }
      if ((goal & 1ull) && !pairTie) {
        const int biA = uniform_i(bi);
        g.set_link<S>(biA, with_flags(g.link<S>(biA), 2u));
        st.lastBest = biA;
        return kAstarGoal;
      }
      // the goal as one of a tied pair: both rows are looked at, the goal's row without its edges
      if (pairTie && (goal & kRows2)) { goalInPair = true; lim = 2; }
      else if (goal) { const int jg = __builtin_ctzll(goal) >> kRowShift; lim = jg < lim ? jg : lim; }
    }
    FM(1);
    const bool rowOn = row < lim;
    const bool act = edgeLane && rowOn;
    uint32_t nb = kNoNb;
    float m0 = 0, m1 = 0, m2 = 0;
    if (act) {
      const AEdge e = edges[ip * kEdgeStride + (uint32_t)el];
      nb = e.nb; m0 = e.mid[0]; m1 = e.mid[1]; m2 = e.mid[2];
    }
    if (__builtin_expect(goalInPair, 0)) nb = ip == endIp ? kNoNb : nb;
    const int bis = rowOn ? bi : 0;
    const uint32_t blink = g.link<S>(bis);
    float b0, b1, b2, bcost;
    uint32_t bparent;
    {
      const int w = bis & (kWindow - 1);
      b0 = L->w_pos[0][w]; b1 = L->w_pos[1][w]; b2 = L->w_pos[2][w]; bcost = L->w_cost[w];
      bparent = L->w_parent[w];
      if (bis < g.nodeCount - kWindow) {   // the node has left the window: rare
        BPSX_KEEP_APART();
        const float4 pc = *reinterpret_cast<const float4*>(g.ws->nodes[bis].pos);   // pos, cost
        b0 = pc.x; b1 = pc.y; b2 = pc.z; bcost = pc.w;
        bparent = g.ws->nodes[bis].parent;
        BPSX_KEEP_APART();
      }
    }
    FM(2);
    // ---- node lookup; the row's own lane hashes its own polygon for the conflict test
    const uint32_t bucket = GeoWave::hash(ownLane ? ip : nb);
    uint32_t chainHead, hitLink;
    int ni = g.find<S>(nb != kNoNb, nb, bucket, &chainHead, &hitLink);
    // the polygon the expanded node was reached from is not entered again
    if (bparent && ni + 1 == (int)bparent) nb = kNoNb;
    FM(3);
    // ---- costs.  A lane without a node to read (idle, or its node is new) reads window slot 127.
    const bool valid = nb != kNoNb;
    const int nis = (valid && ni >= 0) ? ni : 0x7fffffff;
    const int rw = nis & (kWindow - 1);
    uint32_t fl = link_flags(hitLink);
    float p0 = L->w_pos[0][rw], p1 = L->w_pos[1][rw], p2 = L->w_pos[2][rw], oldTotal = L->w_total[rw];
    if (nis < g.nodeCount - kWindow) {   // the node has left the window: rare
      const ANode& hn = g.ws->nodes[nis];
      BPSX_KEEP_APART();
      const float4 pc = *reinterpret_cast<const float4*>(hn.pos);     // pos, cost
      p0 = pc.x; p1 = pc.y; p2 = pc.z; oldTotal = hn.total;
      BPSX_KEEP_APART();
    }
    if (ni < 0) { p0 = m0; p1 = m1; p2 = m2; fl = 0; }   // a new node lies on the portal's midpoint
    const float cx = p0 - b0, cy = p1 - b1, cz = p2 - b2;
    const float ex = e0 - p0, ey = e1 - p1, ez = e2 - p2;
    const float cc = cx * cx + cy * cy + cz * cz, ee = ex * ex + ey * ey + ez * ez;
    float curCost, toEnd;
    sqrt_exact2(cc, ee, &curCost, &toEnd);
    curCost = curCost * 1.0f;
    const bool last = nb == endIp;
    const float cost = last ? bcost + curCost + toEnd * 1.0f : bcost + curCost;
    const float heuristic = last ? 0.0f : toEnd * H_SCALE;
    const float total = cost + heuristic;
    // the total as bits where the lane updates its node, all ones where it does not
    uint32_t tb = (valid && !(fl && total >= oldTotal)) ? __float_as_uint(total) : 0xffffffffu;
    FM(4);
    if (__builtin_expect(goalInPair, 0)) {
      // The goal shares the smallest total with one other node.  If the reference takes the goal
      // first the search ends here; if it takes the other node first, it expands it and ends
      // then.  The path is the goal's node and its ancestors: it is the same both ways when
      // that expansion only creates nodes (none of them can be on the path) and the node pool
      // holds them (an exhausted pool is reported as failure).  Otherwise the heap must say.
      const unsigned long long touches = lanes_where(tb != 0xffffffffu && ni >= 0);
      const int fresh = __popcll(lanes_where(tb != 0xffffffffu));
      if (touches || g.nodeCount + fresh > kMaxNodes) return kAstarTie;
      const int biG = (int)rlane((uint32_t)bi, first_lane(goal & kRows2));
      g.set_link<S>(biG, with_flags(g.link<S>(biG), 2u));
      st.lastBest = biG;
      return kAstarGoal;
    }
    // ---- how many rows stand
    int c = lim;
    bool pairFails = false;
    if (lim > 1) {
      // the first entry j that an update of a row before it reaches or undercuts: the smallest
      // updated total of every row, then of all rows up to it (a scan over the rows), and entry j's
      // lane compares its total with that of the rows before j
      uint32_t low = tb;   // all ones where the lane updates nothing
      low = umin_dpp<0xb1, 0xf>(low);    // quad_perm [1,0,3,2]
      low = umin_dpp<0x4e, 0xf>(low);    // quad_perm [2,3,0,1]
      low = umin_dpp<0x141, 0xf>(low);   // row_half_mirror: every lane has its row's smallest
      low = umin_dpp<0x118, 0xf>(low);   // row_shr:8: odd rows, with the row before
      low = umin_dpp<0x142, 0xa>(low);   // row_bcast:15 into the second and fourth 16 lanes
      low = umin_dpp<0x143, 0xc>(low);   // row_bcast:31 into the upper 32 lanes
      uint32_t before = (uint32_t)__builtin_amdgcn_ds_bpermute((lane - 1) * (kRowLanes * 4), (int)low);
      // a tied pair: both its rows must lie above entry 1's total
      if (__builtin_expect(pairTie, 0)) before = lane == 1 ? rlane(low, kRowLanes) : before;
      const unsigned long long reached = lanes_where(before <= ol.t[0]) & (rows_below(1) & ~1ull);
      const int jv = reached ? __builtin_ctzll(reached) : kRows;
      c = jv < c ? jv : c;
      // conflicts: the earliest row that updates a polygon leaves its mark (pass, row) at the
      // polygon's hash, later rows look for it: a mark of this pass is base + row
      g.tagNow--;
      const uint32_t base = g.tagNow << 3;
      const uint32_t slot = bucket & (uint32_t)(kTagSlots - 1);
      if (tb != 0xffffffffu) atomicMin(&L->tag[slot], base | (uint32_t)row);
      wave_sync();
      const uint32_t seen = L->tag[slot] - base;   // the marking row, or something above 7
      // an earlier row's update matters to a row only at its own node and at the polygons it
      // updates itself: where it reads and leaves alone (a total no better than the node's), a
      // total lowered further changes nothing
      const uint32_t seenr = (tb != 0xffffffffu || (ownLane && rowOn)) ? seen : 0xffffffffu;
      const uint32_t jc = (uint32_t)first_lane(lanes_where(seenr < (uint32_t)row)) >> kRowShift;   // none: far above kRows
      c = jc < (uint32_t)c ? (int)jc : c;
      // rows 0 and 1 of a tied pair in either order: row 0 must not read what row 1 updates either
      if (__builtin_expect(pairTie, 0)) {
        pairFails = c < 2 || (lanes_where(seenr == 1u) & kRows1) != 0;
        if (pairFails && jv >= 2) {
          // The marks are kept per polygon hash, and a pair that fails costs a replay of the log:
          // the polygons that either row updates are compared with those the other row reads,
          // and a clash that was two polygons with one hash lets the pair (and only it) stand.
          const uint32_t readPoly = ownLane ? (rowOn ? ip : 0xffffffffu) : (tb != 0xffffffffu ? nb : 0xffffffffu);
          unsigned long long w = lanes_where(tb != 0xffffffffu) & kRows2;
          bool real = false;
          while (w) {
            const int src = first_lane(w);
            w = without_lane(w, src);
            const unsigned long long others = src < kRowLanes ? (kRows2 & ~kRows1) : kRows1;
            if (lanes_where(readPoly == rlane(nb, src)) & others) real = true;
          }
          if (!real) { pairFails = false; c = 2; }
        }
      }
    }
    if (__builtin_expect(pairFails, 0)) return kAstarTie;
    FM(5);
    const bool rowIn = row < c;
    tb = rowIn ? tb : 0xffffffffu;
    const bool update = tb != 0xffffffffu;
    const bool isNew = update && ni < 0;   // a new node is always taken
    unsigned long long upd = lanes_where(tb != 0xffffffffu);
    // nothing has changed yet: a list that would outgrow its registers goes on in the wider instantiation
    if (__builtin_expect(ol.size - c + __popcll(upd) > 64 * P, 0)) return kAstarGrowHeap;
    (*pops) += (uint32_t)c;
    // the committed rows' nodes are closed
    if (el == 0 && rowIn) g.set_link<S>(bi, with_flags(blink, 2u));
    FM(6);
    // ---- new nodes take consecutive indices in row and edge order
    {
      const unsigned long long need = lanes_where((update ? ni : 0) < 0);
      if (need) {
        const int rank = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(need >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)need, 0u));
        const int count = __popcll(need);
        const int want = g.nodeCount + count;
        // the reference carries on without the nodes that do not fit, but reports anything found
        // after that as failure (only plain DT_SUCCESS counts, PathFinder.cpp:506): stop
        if (S && want > kMaxNodes) { st.outOfNodes = true; return kAstarEmpty; }
        if (isNew) ni = g.nodeCount + rank;
        g.nodeCount = want;
        bool pending = isNew;
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
          if (!lanes_where(pending)) break;
        }
      } else {
        wave_sync();   // the closing writes above stay ahead of the link updates below
      }
    }
    FM(7);
    if (update) {
      ANode& hn = g.ws->nodes[ni];
      const int w = ni & (kWindow - 1);
      const uint32_t parent = (uint32_t)bi + 1u;
      if (!isNew) g.set_link<S>(ni, with_flags(hitLink, 1u));   // open (again)
      if (g.in_window(ni)) {
        L->w_pos[0][w] = p0; L->w_pos[1][w] = p1; L->w_pos[2][w] = p2;
        L->w_cost[w] = cost; L->w_total[w] = total;
        L->w_parent[w] = (uint16_t)parent;
      }
      *reinterpret_cast<float4*>(hn.pos) = make_float4(p0, p1, p2, cost);
      *reinterpret_cast<uint2*>(&hn.total) = make_uint2(tb, parent);
      g.ws->parents[ni] = (uint16_t)parent;
    }
    wave_sync();
    FM(8);
    // ---- the open list: the committed entries leave, the updates enter
    ol.template drop_front<P>(c, lane);
    const uint32_t packed = (uint32_t)ni | (nb << 11);
    {
      // the pass in the operation log: the header from an idle lane, the updates in lane order
      const int rank = (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(upd >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)upd, 0u));
      const bool header = lane == kRowLanes - 1;   // idle: neither an edge's lane nor the node's own
      const int nrec = __popcll(upd);
      if (update || header) {
        OpRec r;
        r.key = header ? ((uint32_t)c | ((uint32_t)nrec << 8)) : tb;
        r.word = header ? (pairTie ? (kOpHeader | kOpUnordered | rlane(cand, 0)) : kOpHeader)
                        : (packed | ((uint32_t)row << 26) | ((fl & 1u) << 29));
        g.ws->oplog[st.logEnd + (header ? 0 : 1 + rank)] = r;
      }
      st.logEnd += 1 + nrec;
    }
    FM(9);
    while (upd) {
      const int src = first_lane(upd);
      upd = without_lane(upd, src);
      ol.template update<P>(rlane(packed, src), rlane(tb, src), lane);
    }
    ol.template count<P>();
    FM(10);
  }
}

// Runs A* for one query. Returns the corridor length (corridor written to F->corridor), or 0
// when the reference would report anything but plain DT_SUCCESS.
BPSX_DEV int astar(GeoWave& g, FunnelLds* F, const NavData& nav, const SceneDev& s, uint32_t startIp, uint32_t endIp,
                   const float* startPos, const float* endPos, uint32_t* pops) {
  const int lane = g.lane;
  if (startIp == endIp) {
    if (lane == 0) F->corridor[0] = (uint16_t)startIp;
    wave_sync();
    return 1;
  }
  AstarState st;
  const AEdge* edges = nav.aedges + (size_t)(uint32_t)uniform_i((int)s.poly_base) * kEdgeStride;
#define ASTAR_ARGS g, st, edges, endIp, endPos, pops
  const uint32_t pops0 = *pops;
  AstarExit ex;
  bool exact = false;   // first with the sorted open list; with the exact loops when that cannot go on
  for (;;) {
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
      g.ws->parents[0] = 0;
      L->w_parent[0] = 0;
      L->n_link[0] = make_link(startIp, 1u, kChainEnd);   // open
      L->first[GeoWave::hash(startIp)] = 0;
    }
    wave_sync();
    st.lastBest = 0;
    st.outOfNodes = false;
    st.rh.init(lane);
    st.rh.push(__float_as_uint(total), startIp << 11, lane);
    bool spill = false, wide = false;
    if (!exact) {
#ifdef BPSX_PHASE_TIMING
      g.phase_t0 = __builtin_readcyclecounter();
#endif
      st.ol.init();
      st.ol.template update<1>(startIp << 11, __float_as_uint(total), lane);
      st.ol.template count<1>();
      st.logEnd = st.synced = 0;
      // the loop is instantiated for links in LDS only or spilling, and for a list within one
      // register pair or two; a search moves on when one more pass could outgrow what it runs in
      bool resolved = false, restart = false;
      int pairs = 1;   // register pairs of the list in use
      for (;;) {
#define BPSX_FAST_RUN(SP) (pairs == 1 ? astar_fast<SP, 1>(g, st, edges, endIp, endPos, pops, resolved) : \
                           pairs == 2 ? astar_fast<SP, 2>(g, st, edges, endIp, endPos, pops, resolved) : \
                                        astar_fast<SP, 4>(g, st, edges, endIp, endPos, pops, resolved))
        ex = spill ? BPSX_FAST_RUN(true) : BPSX_FAST_RUN(false);
#undef BPSX_FAST_RUN
        resolved = false;
        if (ex == kAstarGrowLinks) { g.linkSpills++; spill = true; continue; }
        if (ex == kAstarGrowHeap && pairs < OpenList::kPairs) {
          // the list grows into further registers, empty so far
          if (pairs == 1) { st.ol.clear_pair(1); pairs = 2; }
          else { st.ol.clear_pair(2); st.ol.clear_pair(3); pairs = 4; }
          continue;
        }
        // a list beyond the registers or a full log (neither met in the benchmark configurations'
        // mazes and rooms, both in a hall without obstacles): the search runs again with the exact loops
        if (ex == kAstarGrowHeap || ex == kAstarLogFull) { restart = true; break; }
        if (ex != kAstarTie) break;
        __builtin_amdgcn_s_setprio(3);   // a search that pays for a replay is late from here on
        // a tie: the reference pops what its heap has at the root, so the heap is brought up to
        // date from the log, and that entry goes first
        if (!replay_log(g.ws->oplog, st, lane) || st.rh.size != st.ol.size) { restart = true; break; }
        g.tieReplays++;
        const uint32_t root = rlane(st.rh.n0, 1);
        const unsigned long long at = lanes_where(st.ol.n[0] == root);
        const int p = at ? __ffsll((long long)at) - 1 : -1;
        if (p < 0 || rlane(st.ol.t[0], p) != rlane(st.ol.t[0], 0)) { restart = true; break; }
        const uint32_t front = rlane(st.ol.n[0], 0);
        st.ol.n[0] = wlane(st.ol.n[0], root, 0);
        st.ol.n[0] = wlane(st.ol.n[0], front, p);
        resolved = true;
      }
      if (restart) {
        g.exactRuns++;
        *pops = pops0;
        exact = true;
        continue;
      }
      break;
    }
    {
      wide = false;
      for (;;) {
        if (!spill) ex = wide ? astar_loop2<false, true>(ASTAR_ARGS) : astar_loop2<false, false>(ASTAR_ARGS);
        else ex = wide ? astar_loop2<true, true>(ASTAR_ARGS) : astar_loop2<true, false>(ASTAR_ARGS);
        if (ex == kAstarGrowLinks) { g.linkSpills++; spill = true; }
        else if (ex == kAstarGrowHeap && !wide) wide = true;
        else break;
      }
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
      ex = astar_loop(ASTAR_ARGS);
    }
    break;
  }
#undef ASTAR_ARGS
  // an open list that ran empty, or a pool that ran out, is DT_PARTIAL_RESULT or
  // DT_OUT_OF_NODES in the reference: no path to build, the result is a failure
  if (ex != kAstarGoal || st.outOfNodes) return 0;
  const int lastBest = st.lastBest;
  // getPathToNode: a walk up the parents notes the node indices, then all lanes fill the corridor,
  // which overlays the hash heads; the links stay readable while it is written.  The walk is a
  // chain of dependent reads, 70 of them on average: the parent indices, which HBM also holds
  // side by side, are first copied into the window's arrays (no longer needed), so that the
  // chain runs in LDS; a node beyond what fits there is read from HBM.
  static_assert(offsetof(GeoLds, w_cost) == offsetof(GeoLds, w_total) + sizeof(GeoLds::w_total) &&
                offsetof(GeoLds, w_pos) == offsetof(GeoLds, w_cost) + sizeof(GeoLds::w_cost), "the window's arrays must be contiguous");
  constexpr int kParentsLds = (int)((sizeof(GeoLds::w_total) + sizeof(GeoLds::w_cost) + sizeof(GeoLds::w_pos)) / sizeof(uint16_t));
  static_assert(sizeof(GeoLds::tag) >= kMaxPath * sizeof(uint16_t), "the walk must fit the array it reuses");
  uint16_t* lparent = reinterpret_cast<uint16_t*>(g.L->w_total);
  uint16_t* walk = reinterpret_cast<uint16_t*>(g.L->tag);
  wave_sync();
  const int inLds = g.nodeCount < kParentsLds ? g.nodeCount : kParentsLds;
  {
    const uint32_t* src = reinterpret_cast<const uint32_t*>(g.ws->parents);
    uint32_t* dst = reinterpret_cast<uint32_t*>(lparent);
    for (int i = lane; i < (inLds + 1) / 2; i += 64) dst[i] = src[i];
  }
  wave_sync();
  int length = 0;
  for (int c = lastBest + 1; c && length <= kMaxNodes;) {
    if (lane == 0 && length < kMaxPath) walk[length] = (uint16_t)(c - 1);
    length++;
    c = c - 1 < inLds ? uniform_i((int)lparent[c - 1]) : uniform_i((int)g.ws->parents[c - 1]);
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
  if (lanes_where(missing)) return INF;
  float cs[3], ce[3];
  closest_on_poly_boundary(nav.polys[s.poly_base + F->corridor[0]], startPos, cs);
  closest_on_poly_boundary(nav.polys[s.poly_base + F->corridor[n - 1]], endPos, ce);
  // straight-path points are only needed pairwise: keep the last one and the running length.
  // Every lane computes the same values; the conditions are taken through a ballot so that the
  // control flow is the scalar unit's (no lane masks, no copies at the joins).
  auto all = [](bool b) { return lanes_where(b) != 0; };
  float last[3] = {cs[0], cs[1], cs[2]};
  int npts = 1;
  float length = 0.0f;
  bool finished = false, overflow = false;
  auto append = [&](const float* p, bool isEnd) {
    if (all(vequal(last, p))) return;  // merged with the previous point
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
          if (all(dist_pt_seg_sqr2d(apex[0], apex[2], left, right, t) < 0.001f * 0.001f)) continue;
        }
      } else {
        left[0] = right[0] = ce[0]; left[1] = right[1] = ce[1]; left[2] = right[2] = ce[2];
      }
      if (all(tri_area2d(apex, pr, right) <= 0.0f)) {
        if (all(vequal(apex, pr)) || all(tri_area2d(apex, pl, right) > 0.0f)) {
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
      if (all(tri_area2d(apex, pl, left) >= 0.0f)) {
        if (all(vequal(apex, pl)) || all(tri_area2d(apex, pr, left) < 0.0f)) {
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
BPSX_DEV float geodesic_query(GeoWave& g, const NavData& nav, const GeoQuery& q, uint32_t* pops, uint32_t* corridor) {
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
  const int n = astar(g, F, nav, s, sIp, eIp, q.a, q.b, pops);
  if (n <= 0) return INF;
  *corridor += (uint32_t)n;
  const float len = funnel_length(g.lane, F, nav, s, n, q.a, q.b);
  return len;
}

}  // namespace BPSX_GEO_NS
}  // namespace bpsx
