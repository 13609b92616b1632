// Compile-time geometry shared by the host-side planner (plain C++, no HIP) and the kernels.
#pragma once

namespace hw {

constexpr int MAXF = 64;       // fragments per launch (table travels in the kernel arguments)
constexpr int TILE = 32;       // tokens per wave step
constexpr int NWAVES = 4;      // waves per workgroup
constexpr int NTHREADS = NWAVES * 64;
constexpr int WIDE_ROW_BLOCKS = 8;   // 16-row blocks of a workgroup of the many-rows kernel (32 rows per wave)
constexpr int PAGED_WIDE_MAX_BLOCKS = 8192;   // block-table entries of one sequence the many-rows paged kernel keeps in LDS
constexpr int MAX_SPLITS = 256;  // workgroups per kv head (size of the boundary table below)
// packed-query launches of the many-rows paged kernel whose split is decided on the device (plan_slot)
constexpr int PLAN_SLOT_ROWS = 128;     // rows of a workgroup slot = rows of the widest workgroup
constexpr int PLAN_MAX_GROUPS = 256;    // sequences, and row groups, such a launch takes (one thread of a workgroup each)

}  // namespace hw
