// On-disk navmesh format consumed by the engine: the ".navmesh" file written by
// habitat-sim's PathFinder::saveNavMesh (reference: PathFinder.cpp:259-272, 410-450),
// i.e. an 'MSET' container of Detour tile blobs (DetourNavMesh.h:155-312,
// DetourNavMesh.cpp:970-989 for the section order).  These structs describe bytes
// on disk; nothing here is executable logic.
#pragma once
#include <cstdint>

namespace bpsx {

constexpr int32_t kMsetMagic = ('M' << 24) | ('S' << 16) | ('E' << 8) | 'T';
constexpr int32_t kMsetVersion = 1;
constexpr int32_t kTileMagic = ('D' << 24) | ('N' << 16) | ('A' << 8) | 'V';
constexpr int32_t kTileVersion = 7;
constexpr int kMaxVertsPerPoly = 6;
constexpr uint16_t kExtLink = 0x8000;
constexpr uint32_t kNullLink = 0xffffffffu;
constexpr uint16_t kPolyFlagWalk = 0x01;      // PathFinder.cpp:231-236
constexpr uint16_t kPolyFlagDisabled = 0x04;  // PathFinder.cpp:234

#pragma pack(push, 1)
struct MsetParams {  // dtNavMeshParams
  float orig[3];
  float tileWidth;
  float tileHeight;
  int32_t maxTiles;
  int32_t maxPolys;
};
struct MsetHeader {  // NavMeshSetHeader, 40 bytes
  int32_t magic;
  int32_t version;
  int32_t numTiles;
  MsetParams params;
};
struct MsetTileHeader {  // NavMeshTileHeader, 8 bytes
  uint32_t tileRef;
  int32_t dataSize;
};
struct TileHeader {  // dtMeshHeader, 100 bytes
  int32_t magic;
  int32_t version;
  int32_t x, y, layer;
  uint32_t userId;
  int32_t polyCount;
  int32_t vertCount;
  int32_t maxLinkCount;
  int32_t detailMeshCount;
  int32_t detailVertCount;
  int32_t detailTriCount;
  int32_t bvNodeCount;
  int32_t offMeshConCount;
  int32_t offMeshBase;
  float walkableHeight;
  float walkableRadius;
  float walkableClimb;
  float bmin[3];
  float bmax[3];
  float bvQuantFactor;
};
struct TilePoly {  // dtPoly, 32 bytes
  uint32_t firstLink;
  uint16_t verts[kMaxVertsPerPoly];
  uint16_t neis[kMaxVertsPerPoly];
  uint16_t flags;
  uint8_t vertCount;
  uint8_t areaAndType;
};
struct TileLink {  // dtLink, 12 bytes (contents rebuilt at load; only the space is on disk)
  uint32_t ref;
  uint32_t next;
  uint8_t edge, side, bmin, bmax;
};
struct TilePolyDetail {  // dtPolyDetail, 12 bytes incl. 2 pad
  uint32_t vertBase;
  uint32_t triBase;
  uint8_t vertCount;
  uint8_t triCount;
  uint8_t pad[2];
};
struct TileBVNode {  // dtBVNode, 16 bytes
  uint16_t bmin[3];
  uint16_t bmax[3];
  int32_t i;
};
struct TileOffMeshCon {  // dtOffMeshConnection, 36 bytes
  float pos[6];
  float rad;
  uint16_t poly;
  uint8_t flags, side;
  uint32_t userId;
};
#pragma pack(pop)

static_assert(sizeof(MsetHeader) == 40, "MSET header");
static_assert(sizeof(TileHeader) == 100, "tile header");
static_assert(sizeof(TilePoly) == 32, "poly");
static_assert(sizeof(TileLink) == 12, "link");
static_assert(sizeof(TilePolyDetail) == 12, "detail");
static_assert(sizeof(TileBVNode) == 16, "bv");
static_assert(sizeof(TileOffMeshCon) == 36, "offmesh");

inline int align4(int x) { return (x + 3) & ~3; }
inline size_t align4(size_t x) { return (x + 3) & ~(size_t)3; }
inline uint32_t nextPow2(uint32_t v) {
  v--; v |= v >> 1; v |= v >> 2; v |= v >> 4; v |= v >> 8; v |= v >> 16; v++;
  return v;
}
inline uint32_t ilog2(uint32_t v) {
  uint32_t r = 0;
  while (v >>= 1) r++;
  return r;
}

}  // namespace bpsx
