// Argument validation and split planning of the Hogwild! attention library: pure host code that runs before any HIP
// call, so that every rejection and every plan can be tested (and fuzzed under sanitizers) on a machine without a GPU.
#include "hogwild_plan.h"

#include <cmath>
#include <cstring>

#include "hogwild_consts.h"

namespace hw {
namespace host {

unsigned magic_of(int d) { return (unsigned)(((1ull << 32) + (unsigned long long)d - 1) / (unsigned long long)d); }

// mulhi(n, m) with m = ceil(2^32 / d) = (2^32 + e) / d, 0 <= e < d, is floor(n/d + n e / (d 2^32)): exact as long as
// n e < 2^32 (the second term then cannot carry the sum over the next integer).
bool magic_exact(unsigned long long d, unsigned long long n_max) {
    if (d <= 1) return true;
    const unsigned long long m = ((1ull << 32) + d - 1) / d;
    const unsigned long long e = m * d - (1ull << 32);
    return e == 0 || n_max < ((1ull << 32) + e - 1) / e;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

size_t elem_size(int dtype) { return dtype == HW_F32 ? 4 : 2; }

int validate(const hw_problem* p, int fused) {
    if (p == nullptr) return HW_ERR_NULL;
    if (p->dtype != HW_F32 && p->dtype != HW_F16 && p->dtype != HW_BF16) return HW_ERR_DTYPE;
    if (p->F < 1 || p->F > HW_MAX_FRAGMENTS) return HW_ERR_FRAGMENTS;
    if (p->variant != HW_VARIANT_MFMA && p->variant != HW_VARIANT_VALU_QK) return HW_ERR_UNSUPPORTED;
    if (p->W < 1 || p->Hq < 1 || p->Hkv < 1 || p->S < 1 || p->E < 1 || p->Ev < 1) return HW_ERR_SHAPE;
    if (p->Hq % p->Hkv != 0) return HW_ERR_SHAPE;
    if (!(p->scale > 0.f) || !std::isfinite(p->scale)) return HW_ERR_SHAPE;   // the row max is taken before scaling
    if (fused) {
        if (p->RotE < 0 || p->RotE > p->E || (p->RotE & 1)) return HW_ERR_SHAPE;
    }
    if (p->out == nullptr || p->q == nullptr || p->locations == nullptr) return HW_ERR_NULL;
    if (p->k == nullptr || p->v == nullptr || p->len == nullptr) return HW_ERR_NULL;
    if (fused && p->RotE > 0 && (p->cosines == nullptr || p->sines == nullptr)) return HW_ERR_NULL;
    if (p->len_dev != nullptr && (!fused || p->RotE != p->E)) return HW_ERR_UNSUPPORTED;   // fused entry, full rotary width only
    // one launch only: device-resident lengths (a captured step is one attention launch) and the VALU-logits variant
    if (p->F > HW_MAX_LAUNCH_FRAGMENTS && (p->len_dev != nullptr || p->variant != HW_VARIANT_MFMA)) return HW_ERR_UNSUPPORTED;
    long long rows = (long long)p->W * p->S * (p->Hq / p->Hkv);
    if (rows >= (1 << 20) || p->S >= (1 << 12) || p->Hq / p->Hkv >= (1 << 12)) return HW_ERR_SHAPE;
    if ((long long)p->Hkv * ((rows + 15) / 16) * HW_MAX_SPLITS >= (1 << 20)) return HW_ERR_SHAPE;   // grid size
    for (int f = 0; f < p->F; ++f) {
        if (p->len[f] < 0) return HW_ERR_SHAPE;
        if (p->cap != nullptr && p->cap[f] < p->len[f]) return HW_ERR_SHAPE;
        if (p->len[f] > 0 && (p->k[f] == nullptr || p->v[f] == nullptr)) return HW_ERR_NULL;
        if (!aligned16(p->k[f]) || !aligned16(p->v[f])) return HW_ERR_ALIGN;
        // one kv head of a fragment is addressed through a 32-bit buffer offset
        if ((long long)p->len[f] * (p->E > p->Ev ? p->E : p->Ev) * (long long)elem_size(p->dtype) >= 0x7fff0000ll) return HW_ERR_SHAPE;
    }
    if (!aligned16(p->out) || !aligned16(p->q)) return HW_ERR_ALIGN;
    if (fused && (!aligned16(p->cosines) || !aligned16(p->sines) || !aligned16(p->rq))) return HW_ERR_ALIGN;
    // kernels are instantiated for these head dims (never a silent no-op as in kernel_v21.cuh:992-995)
    if (p->E != p->Ev || (p->E != 64 && p->E != 128 && p->E != 256)) return HW_ERR_UNSUPPORTED;
    if (p->E == 256 && p->variant != HW_VARIANT_MFMA) return HW_ERR_UNSUPPORTED;
    return HW_OK;
}

int make_plan(const hw_problem* p, int num_cus, hw_plan* plan, int fused) {
    if (plan == nullptr) return HW_ERR_NULL;
    if (num_cus < 1) return HW_ERR_SHAPE;
    std::memset(plan, 0, sizeof(*plan));
    // the same limits as validate(): the planner is also reachable on its own (hw_plan_debug)
    if (p->F < 1 || p->F > HW_MAX_LAUNCH_FRAGMENTS) return HW_ERR_FRAGMENTS;
    if (p->W < 1 || p->Hq < 1 || p->Hkv < 1 || p->S < 1 || p->Ev < 1 || p->Hq % p->Hkv != 0 || p->len == nullptr) return HW_ERR_SHAPE;
    const long long rows_ll = (long long)p->W * p->S * (p->Hq / p->Hkv);
    if (rows_ll >= (1 << 20) || p->S >= (1 << 12) || p->Hq / p->Hkv >= (1 << 12)) return HW_ERR_SHAPE;
    if ((long long)p->Hkv * ((rows_ll + 15) / 16) * HW_MAX_SPLITS >= (1 << 20)) return HW_ERR_SHAPE;   // grid size
    const int rows = (int)rows_ll;
    plan->rows = rows;
    // up to 16 rows: one 16-row block per workgroup (two workgroups per CU); up to 96: two blocks, rows beyond 32 in
    // further row groups that read the same KV; more: 128-row workgroups whose waves share every K/V tile through
    // LDS (16-bit types, lengths known on the host) -- a CU can take in about 16 B/clk, so what counts is that every
    // CU reads every byte once
    const bool wide_ok = p->dtype != HW_F32 && p->len_dev == nullptr && p->variant == HW_VARIANT_MFMA && p->E <= 128;
    plan->row_blocks = rows <= 16 ? 1 : 2;
    if (wide_ok && rows > 96) plan->row_blocks = hw::WIDE_ROW_BLOCKS;   // measured crossover: 95 rows 19.2 (narrow) / 19.9 us, 120 rows 21.8 / 20.6 us
    if (p->row_blocks == 1 || p->row_blocks == 2 || (p->row_blocks == hw::WIDE_ROW_BLOCKS && wide_ok)) plan->row_blocks = p->row_blocks;
    // head dimension 256: kernels with one 16-row block only (two blocks of 256-wide accumulators do not fit the registers)
    if (p->E > 128) plan->row_blocks = 1;
    const bool wide = plan->row_blocks == hw::WIDE_ROW_BLOCKS;
    const int rows_per_wg = 16 * plan->row_blocks;
    plan->row_groups = (rows + rows_per_wg - 1) / rows_per_wg;
    plan->tile_tokens = hw::TILE;
    long long tiles = 0;
    for (int f = 0; f < p->F; ++f) {
        if (p->len[f] < 0) return HW_ERR_SHAPE;
        plan->tile_begin[f] = (int)tiles;
        tiles += ((long long)p->len[f] + hw::TILE - 1) / hw::TILE;
        if (tiles > (1ll << 30)) return HW_ERR_SHAPE;
    }
    for (int f = p->F; f <= HW_MAX_LAUNCH_FRAGMENTS; ++f) plan->tile_begin[f] = (int)tiles;
    plan->tiles_per_head = (int)tiles;

    // Split-K policy: fill every CU with its resident workgroups once, but at least one tile per wave
    // in every workgroup, and never more workgroups than tiles.
    int wgs = p->splits;
    if (wgs <= 0) {
        // the two-row-block and fp32 kernels are built for one wave per SIMD (one workgroup per CU)
        const int per_cu = (plan->row_blocks == 1 && p->dtype != HW_F32 && p->E <= 128) ? 2 : 1;
        const int target = per_cu * num_cus;
        wgs = target / (p->Hkv * plan->row_groups);
        // narrow kernels deal a workgroup's tiles to its four waves; in the wide kernel the whole workgroup takes every tile
        const int by_work = wide ? (int)((tiles + 3) / 4) : (int)((tiles + hw::NWAVES - 1) / hw::NWAVES);
        if (wgs > by_work) wgs = by_work;
        // Small problems in 16-bit types: one workgroup per kv head (and row group) holds whole rows, writes the result
        // itself and saves the merge launch (~2.4 us), which is worth more than what the split buys as long as its
        // fragments, opened one after the other, stay few: measured, single fragments of up to 16 tiles 5.8-7.0 us
        // against 8.0-8.2 us, three fragments of 6 / 8 tiles 8.4 / 8.7 against 8.9, of 15 tiles 9.4 against 7.4.  (The
        // fp32 kernel takes ~1 us per tile and loses beyond the 4 tiles that give one workgroup anyway.)
        int nonempty = 0;
        for (int f = 0; f < p->F; ++f) nonempty += p->len[f] > 0 ? 1 : 0;
        if (!wide && p->dtype != HW_F32 && tiles + 6ll * (nonempty > 0 ? nonempty - 1 : 0) <= 20) wgs = 1;
    }
    if (wgs > (int)tiles) wgs = (int)tiles;
    if (wgs > hw::MAX_SPLITS) wgs = hw::MAX_SPLITS;
    if (wgs < 1) wgs = 1;

    // Workgroup boundaries.  Opening a fragment costs a workgroup a fixed prologue (query rotation, a
    // barrier, a pipeline refill) worth about kOpenCost tiles, so boundaries balance tiles + openings
    // rather than tiles alone: a run of tiny fragments is spread over several workgroups instead of
    // serialising their prologues in one straggler.
    {
        const double kOpenCost = wide ? 2.0 : 6.0;   // in tiles of the kernel's own pace (a wide workgroup takes a tile in one step)
        int nfrag_left = 0;
        for (int f = 0; f < p->F; ++f) nfrag_left += p->len[f] > 0 ? 1 : 0;
        long long tiles_left = tiles;
        int wg = 0;
        double used = 0.0;
        plan->wg_tile_begin[0] = 0;
        for (int f = 0; f < p->F; ++f) {
            const int ft = (int)(((long long)p->len[f] + hw::TILE - 1) / hw::TILE);
            if (ft == 0) continue;
            int t = 0;
            while (t < ft) {
                const int wgs_left = wgs - wg;   // including the current one
                // fair share of what remains, counting one opening per remaining fragment and workgroup
                const double remaining = (double)tiles_left + kOpenCost * (nfrag_left + wgs_left - 1) + used;
                const double target = remaining / wgs_left;
                const double room = target - used - kOpenCost;
                if (room < 1.0 && used > 0.0 && wgs_left > 1) {   // not worth opening this fragment here
                    plan->wg_tile_begin[++wg] = plan->tile_begin[f] + t;
                    used = 0.0;
                    continue;
                }
                int take = (int)(room + 0.5);
                if (take < 1) take = 1;
                if (take > ft - t || wgs_left == 1) take = ft - t;
                used += kOpenCost + take;
                t += take;
                tiles_left -= take;
                if (t < ft) {   // the fragment continues in the next workgroup
                    plan->wg_tile_begin[++wg] = plan->tile_begin[f] + t;
                    used = 0.0;
                }
            }
            --nfrag_left;
        }
        wgs = tiles > 0 ? wg + 1 : 1;
        for (int i = wgs; i <= HW_MAX_SPLITS; ++i) plan->wg_tile_begin[i] = (int)tiles;
    }
    plan->wgs_per_head = wgs;
    plan->workgroups = wgs * p->Hkv * plan->row_groups;
    // the kernel divides with multiply-high by ceil(2^32 / d): workgroup id by row groups, (head, split) pair by
    // workgroups per head, row by GQA ratio, (worker, token) by S.  Refuse what that would get wrong.
    if (!magic_exact((unsigned long long)plan->row_groups, (unsigned long long)plan->workgroups) ||
        !magic_exact((unsigned long long)wgs, (unsigned long long)wgs * p->Hkv) ||
        !magic_exact((unsigned long long)(p->Hq / p->Hkv), (unsigned long long)rows + 32) ||
        !magic_exact((unsigned long long)p->S, (unsigned long long)p->W * p->S + 32))
        return HW_ERR_SHAPE;
    const size_t parts = (size_t)p->Hkv * wgs;
    plan->workspace_bytes = parts * rows * ((size_t)p->Ev + 2) * sizeof(float);
    plan->workspace_bytes = (plan->workspace_bytes + 255) & ~(size_t)255;
    // the attention kernel rotates in its prologue only over the full head dimension; any other rotary width
    // goes through the standalone rotation first, into the caller's rq buffer or, without one, into the workspace.
    // Pre-rotated queries (hw_sdpa) never need that: RotE means nothing there.
    if (fused && p->rq == nullptr && p->RotE != p->E && p->RotE >= 0)
        plan->workspace_bytes += ((size_t)p->F * p->W * p->Hq * p->S * p->E * elem_size(p->dtype) + 255) & ~(size_t)255;
    return HW_OK;
}

int plan_call(const hw_problem* p, int num_cus, CallPlan* cp, int fused) {
    if (cp == nullptr || p == nullptr) return HW_ERR_NULL;
    std::memset(cp, 0, sizeof(*cp));
    if (p->F < 1 || p->F > HW_MAX_FRAGMENTS) return HW_ERR_FRAGMENTS;
    if (p->len == nullptr) return HW_ERR_NULL;
    cp->groups = (p->F + HW_MAX_LAUNCH_FRAGMENTS - 1) / HW_MAX_LAUNCH_FRAGMENTS;
    int dummy_rq = 0;
    for (int i = 0; i < cp->groups; ++i) {
        // groups of equal size (130 fragments: 44 + 43 + 43, not 64 + 64 + 2)
        cp->first[i] = (int)(((long long)p->F * i) / cp->groups);
        cp->count[i] = (int)(((long long)p->F * (i + 1)) / cp->groups) - cp->first[i];
        hw_problem q = *p;
        q.F = cp->count[i];
        q.len = p->len + cp->first[i];
        q.cap = p->cap != nullptr ? p->cap + cp->first[i] : nullptr;
        q.rq = &dummy_rq;                      // the room for rotated queries is counted once, below
        const int st = make_plan(&q, num_cus, &cp->plan[i], fused);
        if (st != HW_OK) return st;
        cp->slot_base[i] = cp->slots;
        cp->slots += cp->plan[i].wgs_per_head;
    }
    const size_t rows = (size_t)cp->plan[0].rows;
    cp->partial_bytes = ((size_t)p->Hkv * cp->slots * rows * ((size_t)p->Ev + 2) * sizeof(float) + 255) & ~(size_t)255;
    if (fused && p->rq == nullptr && p->RotE != p->E && p->RotE >= 0)
        cp->rope_bytes = ((size_t)p->F * p->W * p->Hq * p->S * p->E * elem_size(p->dtype) + 255) & ~(size_t)255;
    cp->workspace_bytes = cp->partial_bytes + cp->rope_bytes;
    return HW_OK;
}

int paged_validate(const hw_paged_problem* p) {
    if (p == nullptr) return HW_ERR_NULL;
    if (p->dtype != HW_F32 && p->dtype != HW_F16 && p->dtype != HW_BF16) return HW_ERR_DTYPE;
    if (p->F < 1 || p->F > HW_MAX_FRAGMENTS) return HW_ERR_FRAGMENTS;
    if (p->W < 1 || p->Hq < 1 || p->Hkv < 1 || p->E < 1 || p->Ev < 1) return HW_ERR_SHAPE;
    if (p->Hq % p->Hkv != 0) return HW_ERR_SHAPE;
    if (!(p->scale > 0.f) || !std::isfinite(p->scale)) return HW_ERR_SHAPE;
    const bool varlen = p->cu_seqlens_q != nullptr;
    if (varlen ? p->total_q < 0 : (p->S < 1 || p->S >= (1 << 12))) return HW_ERR_SHAPE;
    if (p->block_size < 1 || p->block_size >= (1 << 12) || p->max_blocks < 1 || p->num_blocks < 1) return HW_ERR_SHAPE;
    if ((long long)p->block_size * p->max_blocks > (1ll << 20)) return HW_ERR_SHAPE;
    if ((long long)p->num_blocks * p->Hkv * p->block_size >= (1ll << 31)) return HW_ERR_SHAPE;
    const long long tokens = varlen ? p->total_q : (long long)p->W * p->S;
    const int gq = p->Hq / p->Hkv;
    if (gq >= (1 << 12) || tokens * gq >= (1 << 20) || p->W >= (1 << 20)) return HW_ERR_SHAPE;
    if (p->out == nullptr || p->q == nullptr || p->locations == nullptr || p->fragment_lengths == nullptr) {
        if (tokens > 0) return HW_ERR_NULL;
    }
    if (p->key_cache == nullptr || p->value_cache == nullptr || p->block_table == nullptr) return HW_ERR_NULL;
    if (!aligned16(p->out) || !aligned16(p->q) || !aligned16(p->key_cache) || !aligned16(p->value_cache)) return HW_ERR_ALIGN;
    if (p->E != p->Ev || (p->E != 64 && p->E != 128 && p->E != 256)) return HW_ERR_UNSUPPORTED;
    if (p->E == 256 && p->dtype == HW_F32) return HW_ERR_UNSUPPORTED;   // the paged kernel's two fp32 K tiles per wave exceed the LDS
    return HW_OK;
}

int paged_plan(const hw_paged_problem* p, int num_cus, hw_paged_plan* plan) {
    if (plan == nullptr) return HW_ERR_NULL;
    if (num_cus < 1) return HW_ERR_SHAPE;
    std::memset(plan, 0, sizeof(*plan));
    const bool varlen = p->cu_seqlens_q != nullptr;
    // the same limits as paged_validate(): the planner is also reachable on its own (hw_paged_plan_debug,
    // hw_paged_workspace_bytes), and the narrowing below must not be handed anything larger
    if (p->W < 1 || p->Hq < 1 || p->Hkv < 1 || p->Ev < 1 || p->Hq % p->Hkv != 0) return HW_ERR_SHAPE;
    if (varlen ? p->total_q < 0 : (p->S < 1 || p->S >= (1 << 12))) return HW_ERR_SHAPE;
    if (p->block_size < 1 || p->block_size >= (1 << 12) || p->max_blocks < 1) return HW_ERR_SHAPE;
    if ((long long)p->block_size * p->max_blocks > (1ll << 20)) return HW_ERR_SHAPE;
    const int gq = p->Hq / p->Hkv;
    const long long tokens = varlen ? p->total_q : (long long)p->W * p->S;
    if (gq >= (1 << 12) || tokens * gq >= (1 << 20) || p->W >= (1 << 20)) return HW_ERR_SHAPE;
    plan->rows = (int)(tokens * gq);
    // rows of one worker share its KV: one 16-row block is enough for plain decoding, two when a worker brings
    // more rows (several query tokens, wide GQA groups)
    const long long rows_per_worker = varlen ? (tokens * gq + p->W - 1) / p->W : (long long)p->S * gq;
    plan->row_blocks = rows_per_worker <= 16 ? 1 : 2;
    // more than one 16-row block per sequence: workgroups of up to 128 rows whose waves share every K/V tile through LDS
    // (16-bit types; the kernel keeps a sequence's block table in LDS, up to PAGED_WIDE_MAX_BLOCKS entries).  Measured on
    // four sequences of 12 528 tokens with 3 / 6 / 12 / 19 query tokens each (15 ... 95 rows per sequence): 36.7 / 36.7 /
    // 45.9 / 69.4 us against 49.4 / 49.5 / 84.6 / 84.7 us of the 32-row workgroups, which stream a sequence's KV once per
    // 32 rows; with one token each (5 rows) the two are equal (36.0 / 36.1 us).
    const bool wide_ok = p->dtype != HW_F32 && p->max_blocks <= hw::PAGED_WIDE_MAX_BLOCKS && p->E <= 128;
    if (wide_ok && rows_per_worker > 16) plan->row_blocks = hw::WIDE_ROW_BLOCKS;
    if (p->row_blocks == 1 || p->row_blocks == 2 || (p->row_blocks == hw::WIDE_ROW_BLOCKS && wide_ok)) plan->row_blocks = p->row_blocks;
    if (p->dtype == HW_F32 || p->E > 128) plan->row_blocks = 1;   // the fp32 and the 256-wide paged kernels exist with one row block only
    const bool wide = plan->row_blocks == hw::WIDE_ROW_BLOCKS;
    const int rpw = 16 * plan->row_blocks;
    long long items;
    if (varlen) items = p->W + tokens * gq / rpw;          // sum_w ceil(rows_w / rpw) <= W + rows / rpw
    else items = (long long)p->W * (((long long)p->S * gq + rpw - 1) / rpw);
    if (items < 1) items = 1;
    plan->row_groups = (int)items;
    if (wide && varlen && p->splits <= 0 && p->W <= hw::PLAN_MAX_GROUPS && items <= hw::PLAN_MAX_GROUPS) {
        // Packed queries in 128-row workgroups: how many rows a sequence brings and how long its KV is are device data,
        // so the device deals the workgroups (every workgroup works out its own share in its prologue):
        // every kv head gets `slots` workgroup slots -- the CUs filled once, a slot per possible row group at least, not
        // more than a slot per four tiles of the longest KV the tables allow -- and each row group takes a share of them
        // in proportion to its work.  A caller that fixes the split (splits > 0) gets the unplanned launch below.
        const long long tiles = ((long long)p->block_size * p->max_blocks + hw::TILE - 1) / hw::TILE;
        const long long fill = num_cus / p->Hkv > 0 ? num_cus / p->Hkv : 1;
        const long long by_work = (long long)p->W * tiles / 4;
        long long slots = fill < by_work ? fill : by_work;
        if (slots < items) slots = items;
        // many possible row groups: the launch oversubscribes the CUs anyway, and slots beyond one per row group are
        // what lets the device cut a long sequence among many short ones
        if (2 * items > fill) slots = items + (fill < by_work ? fill : by_work);
        if (slots >= (1 << 16) || (long long)p->Hkv * slots >= (1 << 20)) return HW_ERR_SHAPE;
        plan->device_planned = 1;
        plan->row_groups = (int)slots;
        plan->splits = 1;
        plan->workgroups = (int)(p->Hkv * slots);
        const unsigned long long positions = (unsigned long long)p->block_size * p->max_blocks + hw::TILE;
        if (!magic_exact((unsigned long long)slots, (unsigned long long)p->Hkv * slots) ||
            !magic_exact((unsigned long long)gq, (unsigned long long)tokens * gq + 32) ||
            !magic_exact((unsigned long long)p->block_size, positions))
            return HW_ERR_SHAPE;
        plan->workspace_bytes = (size_t)p->Hkv * (size_t)slots * hw::PLAN_SLOT_ROWS * ((size_t)p->Ev + 2) * sizeof(float) +
                                (size_t)p->Hkv * (size_t)(plan->rows > 0 ? plan->rows : 1) * 2 * sizeof(int);
        plan->workspace_bytes = (plan->workspace_bytes + 255) & ~(size_t)255;
        return HW_OK;
    }
    int splits = p->splits;
    if (splits <= 0) {
        // The paged kernels run one workgroup per CU.  Few (kv head, row group) pairs: split until every CU has
        // one workgroup.  More pairs than half the CUs: the chip is oversubscribed anyway, and about three
        // workgroups per CU even out the tail between sequences of different length (measured best on packed
        // variable-length queries) -- there a wave keeps at least four tiles.
        const long long pairs = (long long)p->Hkv * items;
        const long long tiles = ((long long)p->block_size * p->max_blocks + hw::TILE - 1) / hw::TILE;
        long long s, by_work;
        if (wide) {
            // every wave takes every tile of its workgroup: fill the CUs once, at least four tiles per workgroup
            s = pairs < num_cus ? num_cus / pairs : 1;
            by_work = (tiles + 3) / 4;
        } else if (2 * pairs <= num_cus) {
            s = num_cus / pairs;
            by_work = (tiles + hw::NWAVES - 1) / hw::NWAVES;
        } else {
            s = (3LL * num_cus + pairs - 1) / pairs;
            by_work = tiles / (4 * hw::NWAVES);
        }
        if (s > by_work) s = by_work;
        splits = (int)s;
    }
    if (splits > 64) splits = 64;
    if (splits < 1) splits = 1;
    plan->splits = splits;
    const long long wgs = (long long)p->Hkv * items * splits;
    if (wgs >= (1 << 20)) return HW_ERR_SHAPE;
    plan->workgroups = (int)wgs;
    // the kernel divides with multiply-high by ceil(2^32 / d): workgroup id by splits, the quotient by row groups, row
    // group by row groups per worker, row by GQA ratio, token by tokens per worker, position by block size.  A large
    // divisor (many sequences) can make that inexact; such a launch is refused instead of decoding wrong indices.
    const unsigned long long positions = (unsigned long long)p->block_size * p->max_blocks + hw::TILE;
    if (!magic_exact((unsigned long long)splits, (unsigned long long)wgs) ||
        !magic_exact((unsigned long long)items, (unsigned long long)p->Hkv * items) ||
        !magic_exact((unsigned long long)(varlen ? 1 : items / p->W), (unsigned long long)items) ||
        !magic_exact((unsigned long long)gq, (unsigned long long)tokens * gq + 32) ||
        !magic_exact((unsigned long long)(varlen ? 1 : p->S), (unsigned long long)tokens + 32) ||
        !magic_exact((unsigned long long)p->block_size, positions))
        return HW_ERR_SHAPE;
    plan->workspace_bytes = (size_t)p->Hkv * splits * (size_t)(plan->rows > 0 ? plan->rows : 1) * ((size_t)p->Ev + 2) * sizeof(float);
    plan->workspace_bytes = (plan->workspace_bytes + 255) & ~(size_t)255;
    return HW_OK;
}

}  // namespace host
}  // namespace hw
