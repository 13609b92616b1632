// Fuzz of the host-only part of the library (inference_lib_amd/csrc/hogwild_plan.cpp): random problems through the
// validators and the two split planners, built with -fsanitize=address,undefined.  Checks, for every plan that is
// accepted, what the kernels rely on: boundaries monotone and covering all tiles, table sizes within their arrays,
// workspace at least what the kernels index, and every multiply-high division exact over its whole range.
// usage: plan_fuzz <iterations> <seed>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "../../inference_lib_amd/csrc/hogwild_consts.h"
#include "../../inference_lib_amd/csrc/hogwild_plan.h"

using namespace hw::host;

static int failures = 0;
#define CHECK(cond, ...)                                                   \
    do {                                                                   \
        if (!(cond)) {                                                     \
            if (failures++ < 20) { std::printf("FAIL %s:%d %s: ", __FILE__, __LINE__, #cond); std::printf(__VA_ARGS__); std::printf("\n"); } \
        }                                                                  \
    } while (0)

static void check_division(unsigned d, unsigned long long n_max, const char* what) {
    const unsigned m = magic_of((int)d);
    for (unsigned long long n = 0; n <= n_max; ++n) {
        const unsigned q = m ? (unsigned)((n * (unsigned long long)m) >> 32) : (unsigned)n;
        if (q != n / d) {
            CHECK(false, "%s: %llu / %u gives %u", what, n, d, q);
            return;
        }
    }
}

static void fuzz_fragments(std::mt19937_64& rng) {
    auto U = [&](long long lo, long long hi) { return (long long)(lo + rng() % (unsigned long long)(hi - lo + 1)); };
    hw_problem p{};
    const int dts[3] = {HW_F32, HW_F16, HW_BF16};
    p.dtype = dts[U(0, 2)];
    p.F = (int)U(1, U(0, 3) == 0 ? HW_MAX_LAUNCH_FRAGMENTS : 12);
    p.Hkv = (int)(U(0, 5) == 0 ? U(1, 64) : (1 << U(0, 3)));
    p.Hq = p.Hkv * (int)(U(0, 9) == 0 ? U(1, 4095) : U(1, 16));
    p.W = (int)(U(0, 9) == 0 ? U(1, 5000) : U(1, 16));
    p.S = (int)(U(0, 9) == 0 ? U(1, 4095) : U(1, 8));
    const int dims[3] = {64, 128, 256};
    p.E = p.Ev = dims[U(0, 2)];
    p.RotE = p.E;
    p.scale = 0.1f;
    p.splits = U(0, 3) == 0 ? (int)U(1, 300) : 0;
    p.row_blocks = (int)(U(0, 6) == 0 ? 8 : U(0, 2));
    std::vector<int32_t> len(p.F);
    for (auto& l : len) {
        switch (U(0, 5)) {
            case 0: l = 0; break;
            case 1: l = (int)U(1, 40); break;
            case 2: l = (int)U(1, 200000); break;
            default: l = (int)U(1, 5000); break;
        }
    }
    p.len = len.data();
    const int cus = (int)(U(0, 3) == 0 ? U(1, 1024) : 256);
    hw_plan plan;
    const int st = make_plan(&p, cus, &plan);
    if (st != HW_OK) {
        CHECK(st == HW_ERR_SHAPE, "make_plan status %d", st);
        return;
    }
    long long tiles = 0;
    for (int f = 0; f < p.F; ++f) {
        CHECK(plan.tile_begin[f] == tiles, "tile_begin[%d]", f);
        tiles += (len[f] + hw::TILE - 1) / hw::TILE;
    }
    for (int f = p.F; f <= HW_MAX_LAUNCH_FRAGMENTS; ++f) CHECK(plan.tile_begin[f] == tiles, "tile_begin tail %d", f);
    const int rows = p.W * p.S * (p.Hq / p.Hkv);
    CHECK(plan.rows == rows && plan.tiles_per_head == tiles, "rows / tiles");
    CHECK(plan.row_blocks == 1 || plan.row_blocks == 2 || plan.row_blocks == 8, "row_blocks %d", plan.row_blocks);
    if (p.E == 256) CHECK(plan.row_blocks == 1, "head dimension 256 planned with %d row blocks", plan.row_blocks);
    if (p.dtype == HW_F32) CHECK(plan.row_blocks != 8, "fp32 planned with 128-row workgroups");
    CHECK((long long)plan.row_groups * 16 * plan.row_blocks >= rows && (long long)(plan.row_groups - 1) * 16 * plan.row_blocks < rows, "row groups");
    const int wgs = plan.wgs_per_head;
    CHECK(wgs >= 1 && wgs <= HW_MAX_SPLITS, "wgs %d", wgs);
    CHECK(plan.workgroups == wgs * p.Hkv * plan.row_groups, "workgroups");
    CHECK(plan.wg_tile_begin[0] == 0, "first boundary");
    for (int g = 0; g < wgs; ++g) {
        CHECK(plan.wg_tile_begin[g] <= plan.wg_tile_begin[g + 1], "boundaries not monotone at %d", g);
        if (tiles >= wgs && p.splits == 0) CHECK(plan.wg_tile_begin[g] < plan.wg_tile_begin[g + 1] || tiles == 0, "empty workgroup %d of %d (tiles %lld)", g, wgs, tiles);
    }
    for (int g = wgs; g <= HW_MAX_SPLITS; ++g) CHECK(plan.wg_tile_begin[g] == tiles, "boundary tail %d = %d, tiles %lld", g, plan.wg_tile_begin[g], tiles);
    const size_t need = (size_t)p.Hkv * wgs * rows * ((size_t)p.Ev + 2) * sizeof(float);
    CHECK(plan.workspace_bytes >= need, "workspace %zu < %zu", plan.workspace_bytes, need);
    // in-kernel divisions over everything the kernel can feed them
    check_division((unsigned)plan.row_groups, (unsigned long long)plan.workgroups - 1, "workgroup id / row groups");
    check_division((unsigned)wgs, (unsigned long long)wgs * p.Hkv - 1, "(head, split) / workgroups per head");
    check_division((unsigned)(p.Hq / p.Hkv), (unsigned long long)rows + 31, "row / gqa");
    check_division((unsigned)p.S, (unsigned long long)p.W * p.S + 31, "(worker, token) / S");
    // the validator must accept or refuse, never crash, whatever the pointers are (it dereferences only the host arrays)
    std::vector<const void*> kp(p.F, (const void*)0x1000), vp(p.F, (const void*)0x2000);
    p.k = kp.data(); p.v = vp.data();
    p.out = (void*)0x100; p.q = (void*)0x200; p.locations = (const int32_t*)0x300; p.cosines = (const float*)0x400; p.sines = (const float*)0x500;
    if (U(0, 4) == 0) kp[U(0, p.F - 1)] = (const void*)0x1001;
    const int vs = validate(&p, (int)U(0, 1));
    CHECK(vs <= 0 && vs >= HW_ERR_STATIC_SCRATCH, "validate status %d", vs);
}

// A whole call: up to HW_MAX_FRAGMENTS fragments in groups of at most HW_MAX_LAUNCH_FRAGMENTS, one launch each.
static void fuzz_call(std::mt19937_64& rng) {
    auto U = [&](long long lo, long long hi) { return (long long)(lo + rng() % (unsigned long long)(hi - lo + 1)); };
    hw_problem p{};
    p.dtype = U(0, 1) ? HW_BF16 : HW_F32;
    p.F = (int)(U(0, 2) == 0 ? U(1, HW_MAX_FRAGMENTS + 2) : U(60, 140));
    p.Hkv = 1 << U(0, 3);
    p.Hq = p.Hkv * (int)U(1, 8);
    p.W = (int)U(1, 70);
    p.S = (int)U(1, 3);
    p.E = p.Ev = U(0, 1) ? 128 : 64;
    p.RotE = U(0, 3) == 0 ? p.E / 2 : p.E;
    p.scale = 0.1f;
    p.splits = U(0, 3) == 0 ? (int)U(1, 300) : 0;
    std::vector<int32_t> len(p.F);
    for (auto& l : len) l = (int)(U(0, 3) == 0 ? 0 : U(1, 700));
    p.len = len.data();
    const int fused = (int)U(0, 1);
    const int cus = (int)(U(0, 3) == 0 ? U(1, 1024) : 256);
    CallPlan cp;
    const int st = plan_call(&p, cus, &cp, fused);
    if (p.F > HW_MAX_FRAGMENTS) {
        CHECK(st == HW_ERR_FRAGMENTS, "plan_call took %d fragments (status %d)", p.F, st);
        return;
    }
    if (st != HW_OK) {
        CHECK(st == HW_ERR_SHAPE, "plan_call status %d", st);
        return;
    }
    CHECK(cp.groups == (p.F + HW_MAX_LAUNCH_FRAGMENTS - 1) / HW_MAX_LAUNCH_FRAGMENTS && cp.groups <= MAX_GROUPS, "groups %d for %d fragments", cp.groups, p.F);
    int next = 0, slots = 0;
    for (int i = 0; i < cp.groups; ++i) {
        CHECK(cp.first[i] == next && cp.count[i] >= 1 && cp.count[i] <= HW_MAX_LAUNCH_FRAGMENTS, "group %d: first %d count %d", i, cp.first[i], cp.count[i]);
        next += cp.count[i];
        CHECK(cp.slot_base[i] == slots, "slot base of group %d", i);
        slots += cp.plan[i].wgs_per_head;
        long long tiles = 0;
        for (int f = 0; f < cp.count[i]; ++f) tiles += (len[cp.first[i] + f] + hw::TILE - 1) / hw::TILE;
        CHECK(cp.plan[i].tiles_per_head == tiles, "tiles of group %d", i);
        CHECK(cp.plan[i].rows == cp.plan[0].rows && cp.plan[i].row_blocks == cp.plan[0].row_blocks, "groups disagree on the rows");
    }
    CHECK(next == p.F && slots == cp.slots, "groups cover %d of %d fragments, %d of %d slots", next, p.F, slots, cp.slots);
    const size_t need = (size_t)p.Hkv * cp.slots * cp.plan[0].rows * ((size_t)p.Ev + 2) * sizeof(float);
    const size_t rope = (fused && p.RotE != p.E) ? (size_t)p.F * p.W * p.Hq * p.S * p.E * (p.dtype == HW_F32 ? 4 : 2) : 0;
    CHECK(cp.partial_bytes >= need && cp.partial_bytes % 256 == 0 && cp.rope_bytes >= rope && cp.workspace_bytes == cp.partial_bytes + cp.rope_bytes,
          "workspace %zu (partials %zu need %zu, rope %zu need %zu)", cp.workspace_bytes, cp.partial_bytes, need, cp.rope_bytes, rope);
    if (cp.groups == 1) {      // a call of one launch is the plan of that launch
        hw_plan plan;
        CHECK(make_plan(&p, cus, &plan, fused) == HW_OK && plan.workspace_bytes == cp.workspace_bytes && plan.wgs_per_head == cp.slots, "single group differs from make_plan");
    }
}

static void fuzz_paged(std::mt19937_64& rng) {
    auto U = [&](long long lo, long long hi) { return (long long)(lo + rng() % (unsigned long long)(hi - lo + 1)); };
    hw_paged_problem p{};
    p.dtype = HW_BF16;
    p.F = (int)U(1, 8);
    p.Hkv = 1 << U(0, 3);
    p.Hq = p.Hkv * (int)U(1, 16);
    p.E = p.Ev = U(0, 2) == 0 ? 256 : 128;
    p.W = (int)(U(0, 3) == 0 ? U(1, 100000) : U(1, 64));
    p.S = (int)U(1, 8);
    p.block_size = (int)(U(0, 3) == 0 ? U(1, 4095) : (1 << U(0, 7)));
    p.max_blocks = (int)U(1, (1 << 20) / p.block_size);
    p.num_blocks = (int)U(1, 1 << 16);
    p.scale = 0.1f;
    p.splits = U(0, 3) == 0 ? (int)U(1, 80) : 0;
    p.row_blocks = (int)(U(0, 4) == 0 ? 8 : U(0, 2));
    const bool varlen = U(0, 1);
    int32_t dummy = 0;
    if (varlen) {
        p.cu_seqlens_q = &dummy;      // only its presence matters to the planner
        p.total_q = (int)U(0, 200000);
    }
    const int cus = (int)(U(0, 3) == 0 ? U(1, 1024) : 256);
    hw_paged_plan plan;
    const int st = paged_plan(&p, cus, &plan);
    {   // sizes beyond the kernels' index ranges are refused by the planner itself
        const long long tk = varlen ? p.total_q : (long long)p.W * p.S;
        if (tk * (p.Hq / p.Hkv) >= (1 << 20) || p.W >= (1 << 20)) CHECK(st == HW_ERR_SHAPE, "paged_plan took %lld rows, %d sequences (status %d)", tk * (p.Hq / p.Hkv), p.W, st);
    }
    if (st != HW_OK) {
        CHECK(st == HW_ERR_SHAPE, "paged_plan status %d", st);
        return;
    }
    const int gq = p.Hq / p.Hkv;
    const long long tokens = varlen ? p.total_q : (long long)p.W * p.S;
    CHECK(plan.rows == tokens * gq, "rows");
    CHECK(plan.splits >= 1 && plan.splits <= 64, "splits %d", plan.splits);
    CHECK(plan.row_groups >= 1, "row groups");
    if (p.E == 256) CHECK(plan.row_blocks == 1 && !plan.device_planned, "head dimension 256 planned with %d row blocks", plan.row_blocks);
    CHECK((long long)plan.workgroups == (long long)p.Hkv * plan.row_groups * plan.splits && plan.workgroups < (1 << 20), "workgroups");
    size_t need = (size_t)p.Hkv * plan.splits * (size_t)(plan.rows > 0 ? plan.rows : 1) * ((size_t)p.Ev + 2) * sizeof(float);
    if (plan.device_planned) {
        // the device deals `row_groups` workgroup slots per kv head: packed queries in 128-row workgroups only, no fixed
        // split, a thread of one workgroup per sequence and per possible row group, a slot per possible row group at
        // least; partial sums by slot, then two ints per row for the merge
        CHECK(varlen && plan.row_blocks == 8 && p.splits <= 0 && plan.splits == 1, "device-planned launch of the wrong kind");
        CHECK(p.W <= hw::PLAN_MAX_GROUPS && plan.row_groups < (1 << 16), "device-planned launch too large");
        CHECK(plan.row_groups >= p.W + tokens * gq / 128, "fewer slots (%d) than possible row groups", plan.row_groups);
        need = (size_t)p.Hkv * plan.row_groups * hw::PLAN_SLOT_ROWS * ((size_t)p.Ev + 2) * sizeof(float) + (size_t)p.Hkv * plan.rows * 2 * sizeof(int);
    }
    CHECK(plan.workspace_bytes >= need, "workspace");
    check_division((unsigned)plan.splits, (unsigned long long)plan.workgroups - 1, "workgroup id / splits");
    check_division((unsigned)plan.row_groups, (unsigned long long)p.Hkv * plan.row_groups - 1, "(head, item) / items");
    if (!varlen) check_division((unsigned)(plan.row_groups / p.W), (unsigned long long)plan.row_groups - 1, "item / row groups per worker");
    check_division((unsigned)gq, (unsigned long long)tokens * gq + 31, "row / gqa");
    if (!varlen) check_division((unsigned)p.S, (unsigned long long)tokens + 31, "token / S");
    check_division((unsigned)p.block_size, (unsigned long long)p.block_size * p.max_blocks + hw::TILE - 1, "position / block size");
}

int main(int argc, char** argv) {
    const long iters = argc > 1 ? std::atol(argv[1]) : 2000;
    const unsigned long long seed = argc > 2 ? std::strtoull(argv[2], nullptr, 10) : 1;
    std::mt19937_64 rng(seed);
    for (long i = 0; i < iters; ++i) {
        fuzz_fragments(rng);
        fuzz_call(rng);
        fuzz_paged(rng);
    }
    // a divisor the multiply-high division gets wrong must be refused: 40 000 decode sequences on 8 kv heads
    {
        hw_paged_problem p{};
        p.dtype = HW_BF16; p.F = 1; p.Hkv = 8; p.Hq = 8; p.E = p.Ev = 128; p.W = 40000; p.S = 1;
        p.block_size = 16; p.max_blocks = 8; p.num_blocks = 1 << 16; p.scale = 0.1f;
        hw_paged_plan plan;
        const int st = paged_plan(&p, 256, &plan);
        CHECK(st == HW_ERR_SHAPE, "inexact division accepted (status %d)", st);
        CHECK(!magic_exact(40000, 8ull * 40000), "magic_exact misses a known counter-example");
    }
    std::printf("%ld iterations, %d failures\n", iters, failures);
    return failures ? 1 : 0;
}
