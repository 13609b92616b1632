// Host-only part of the library: argument validation and split planning.  Plain C++ with no HIP dependency, so it
// builds with any host compiler (the test suite builds it with g++ -fsanitize=address,undefined and fuzzes it).
#pragma once
#include <stddef.h>
#include <stdint.h>

#include "../../include/hogwild_hip.h"

namespace hw {
namespace host {

bool aligned16(const void* p);
size_t elem_size(int dtype);

// ceil(2^32 / d) mod 2^32: the multiplier of the kernels' multiply-high division (0 stands for d == 1)
unsigned magic_of(int d);
// true if floor(n / d) == mulhi(n, magic_of(d)) for every 0 <= n <= n_max
bool magic_exact(unsigned long long d, unsigned long long n_max);

int validate(const hw_problem* p, int fused);
// fused != 0: size the workspace for hw_fused_attention (room for the rotated queries when the rotary width is not the head
// dimension and the caller passes no rq buffer); 0: for hw_sdpa
int make_plan(const hw_problem* p, int num_cus, hw_plan* plan, int fused = 1);
// A call's fragments in groups of at most HW_MAX_LAUNCH_FRAGMENTS, one attention launch each.  Group i takes fragments
// first[i] .. first[i] + count[i] - 1, is planned like a problem of its own (plan[i]; its workspace_bytes is not used) and
// writes its split-K partials into slots slot_base[i] .. slot_base[i] + plan[i].wgs_per_head - 1 of every kv head's
// `slots` slots.
constexpr int MAX_GROUPS = (HW_MAX_FRAGMENTS + HW_MAX_LAUNCH_FRAGMENTS - 1) / HW_MAX_LAUNCH_FRAGMENTS;
struct CallPlan {
    int groups;
    int first[MAX_GROUPS], count[MAX_GROUPS], slot_base[MAX_GROUPS];
    hw_plan plan[MAX_GROUPS];
    int slots;                 // partial slots per kv head over all groups
    size_t partial_bytes;      // part_o + part_ml of all slots
    size_t rope_bytes;         // room for the rotated queries (fused entry, rotary width != head dim, no rq buffer), else 0
    size_t workspace_bytes;    // partial_bytes + rope_bytes
};
int plan_call(const hw_problem* p, int num_cus, CallPlan* cp, int fused);
int paged_validate(const hw_paged_problem* p);
int paged_plan(const hw_paged_problem* p, int num_cus, hw_paged_plan* plan);

}  // namespace host
}  // namespace hw
