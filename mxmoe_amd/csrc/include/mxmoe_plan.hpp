// Layout of the buffer that the device-side planner fills and the planned launches read.
#pragma once
#include "mxmoe_launch.hpp"

namespace mxmoe {

// Layout of the plan buffer (bytes): one FusedArgs per launch (a launch holds at most kMaxProblems problems; a block of more experts is
// run as ceil(Et / kMaxProblems) launches over consecutive chunks of experts), then for all Et experts the quantisers' table
// int64 [4][Et], the pointer arrays void* [5][Et] (A, B, scale_a, scale_b, C), two int64 (rows that were routed; address of the shared
// expert's output rows, 0 if none), and the sizes mxmoe_dim3 [Et].
constexpr size_t kFusedArgsStride = (sizeof(FusedArgs) + 255) & ~(size_t)255;
struct PlanLayout {
  int chunks;
  size_t table, ptrs, misc, sizes, total;
  __host__ __device__ explicit PlanLayout(int et) {
    chunks = et > 0 ? (et + kMaxProblems - 1) / kMaxProblems : 1;
    table = (size_t)chunks * kFusedArgsStride;
    ptrs = table + (size_t)4 * et * 8;
    misc = ptrs + (size_t)5 * et * 8;
    sizes = misc + 16;
    total = (sizes + (size_t)et * sizeof(mxmoe_dim3) + 255) & ~(size_t)255;
  }
};

}  // namespace mxmoe
