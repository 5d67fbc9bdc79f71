// Host-side navmesh ingest: ".navmesh" (MSET) bytes -> the polygon records, BV tree and
// height mesh arrays that get uploaded to HBM.
#pragma once
#include <cstddef>
#include <cstdint>
#include <vector>

#include "device_types.h"

namespace bpsx {

struct HostScene {
  std::vector<PolyRec> polys;     // tri_base / dvert_base are scene-relative until upload
  std::vector<AEdge> aedges;      // [polygon][kEdgeStride]
  std::vector<BVNodeDev> bv;
  std::vector<uint8_t> dtris;     // [.][4]
  std::vector<float> dverts;      // [.][3]
  std::vector<float> episodes;    // [.][10]
  SceneDev dev{};                 // *_base fields are filled by the uploader
};

// Returns BPSX_OK or a negative code (message via bpsx_last_error). Every index the
// kernels later follow is bounds-checked here.
int parse_navmesh(const uint8_t* bytes, size_t n, HostScene* out);

}  // namespace bpsx
