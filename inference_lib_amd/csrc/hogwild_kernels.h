// Internal interface between the C-ABI host code and the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "hogwild_consts.h"

namespace hw {

// Fragment table passed by value in the kernel arguments: no per-call host-to-device copy of a pointer
// table (the reference does one, src/binding.cu:84-103).
struct FragTable {
    const void* k[MAXF];
    const void* v[MAXF];
    struct LenCap {
        int len;                // tokens in the fragment
        int cap;                // rows between consecutive kv heads of the fragment's buffers (>= len; == len when packed)
    } lc[MAXF];                 // one 8-byte load per lane fetches both
    int tile_begin[MAXF + 1];   // prefix sum of ceil(len/TILE): position of each fragment in a head's tile sequence
};

// Scalar arguments of the attention kernel: exactly 32 dwords at the start of the kernel-argument segment
// so that the kernel can fetch all of them with two back-to-back 64-byte scalar loads.
struct alignas(64) KernelHeader {
    const void* q;
    const int* loc;
    const float* cos;
    const float* sin;
    void* rq;
    float* part_o;      // [Hkv][wgs_per_head][R][Ev]  unnormalised partial outputs
    float* part_ml;     // [Hkv][wgs_per_head][R][2]   running max (base-2 units) and sum
    const int* len_dev; // [F] current fragment lengths in device memory, or null: the table's lengths are exact.
                        // With it the table's lengths are the bounds the split was planned for and fragment f holds
                        // min(bound, len_dev[f]) tokens, so a captured launch stays valid while segments grow.
    int F, W, Hq, Hkv, S, R;
    int nrg, wgs_per_head, nwg;
    int slot_stride;    // partial slots per kv head in the workspace: wgs_per_head, or more when the fragments of a call
                        // are spread over several launches that write side by side (part_o / part_ml then point at this
                        // launch's first slot)
    int flags;          // KH_XCD_REMAP | KH_DIRECT | KH_PREROTATED
    float sc;           // scale * log2(e)
    unsigned magic_gq, magic_s, magic_nrg, magic_wg;   // ceil(2^32 / d) for d = Hq/Hkv, S, nrg, wgs_per_head
};
static_assert(sizeof(KernelHeader) == 128, "KernelHeader must be 32 dwords");
constexpr int KH_XCD_REMAP = 1;   // consecutive logical workgroup ids share an XCD (the grid is a multiple of 8)
constexpr int KH_DIRECT = 2;      // one workgroup per kv head and row group: it normalises its own result and writes out / lse
                                  // itself (part_o then holds the address of out, part_ml that of lse or null); no merge launch
constexpr int KH_PREROTATED = 4;  // the queries arrive rotated, [F,W,Hq,S,E] (read by the launchers only)

struct KernelArgs {
    KernelHeader h;
    FragTable frag;
    int wg_tile[MAX_SPLITS + 1];   // first tile of each workgroup of a head (same for all heads)
};

struct MergeArgs {
    const float* part_o;
    const float* part_ml;
    void* out;
    float* lse;
    int W, Hq, Hkv, S, R, wgs_per_head;
    int xcd_local;      // kv head h was computed on XCD h / (Hkv/8): merge it there
    // Partials laid out by workgroup slot instead of by row (the paged launch that is planned on the device, see
    // PagedHeader): row_tab[kv head][r] = {first slot | slots << 16, row within the slot}, a slot holds PLAN_SLOT_ROWS rows, pslots
    // slots per kv head; wgs_per_head then only bounds the slots of a row (for the choice of the merge kernel's shape).
    const int* row_tab;
    int pslots;
};

hipError_t launch_attention(const KernelArgs& ka, int dtype, int E, int rb, int variant, hipStream_t stream);
// many rows per kv head: 128-row workgroups that share every K/V tile through LDS (16-bit types, host-side lengths)
hipError_t launch_attention_wide(const KernelArgs& ka, int dtype, int E, hipStream_t stream);
hipError_t launch_merge(const MergeArgs& ma, int dtype, int EV, hipStream_t stream);
hipError_t launch_rope(void* out, const void* q, const float* cosv, const float* sinv, int dtype, int F, int W, int Hq, int S,
                       int E, int RotE, hipStream_t stream);

// ---- paged variants: KV of worker w lives in blocks of a shared cache, found through a block table ----

// Scalar arguments of the paged attention kernel: 48 dwords, fetched with three 64-byte scalar loads.
// The queries, locations and the output use the layout [LW, Hq, LS]: (W, S) for the fixed-length operator,
// (total_q, 1) for the packed variable-length one.
struct alignas(64) PagedHeader {
    const void* q;             // [F, LW, Hq, LS, E] rotated queries
    const int* loc;            // [F, LW*LS]
    const int* frag_len;       // [F] or, with cu_q, [F, W]
    const void* kcache;        // [num_blocks, Hkv, block_size, E]
    const void* vcache;        // [num_blocks, Hkv, block_size, Ev]
    const int* block_table;    // [W, max_blocks]
    const int* cu_q;           // [W + 1] query-token prefix sums, or null: worker w owns tokens w*LS .. (w+1)*LS-1
    float* part_o;             // [Hkv][nsplit][R][Ev]; planned on the device: [Hkv][nitems][PLAN_SLOT_ROWS][Ev]
    float* part_ml;            // [Hkv][nsplit][R][2];  planned: [Hkv][nitems][PLAN_SLOT_ROWS][2], the merge's row table right behind it
    int F, W, Hq, Hkv, LW, LS;
    int R;                     // LW*LS*(Hq/Hkv): query rows per kv head
    int block_size, max_blocks, num_blocks;
    int nsplit;                // workgroups that share one (kv head, row group)
    int nitems;                // row groups over all workers (an upper bound when cu_q is given)
    int nrg;                   // row groups per worker (fixed-length operator)
    int nwg;
    int flags;                 // PH_*
    float sc;                  // scale * log2(e)
    unsigned magic_gq, magic_ls, magic_bs, magic_nsplit, magic_nitems, magic_nrg;   // ceil(2^32 / d)
    int pad[8];
};
static_assert(sizeof(PagedHeader) == 192, "PagedHeader must be 48 dwords");
constexpr int PH_XCD_REMAP = 1;    // consecutive logical workgroup ids share an XCD
// The launch is planned on the device (packed queries in 128-row workgroups): nsplit = 1, nitems = workgroup slots per
// kv head, and what slot j of a head does -- which row group of which sequence, which share of its tiles -- every
// workgroup works out for itself from the query and KV lengths (plan_slot).  Behind part_ml the workgroups leave the
// merge kernel a table per kv head of where each row's partial sums lie (MergeArgs::row_tab).
constexpr int PH_PLANNED = 2;

struct CopyBlocksArgs {
    const void* key_states;    // [B, Hkv, S_new, E]   (element strides below, innermost contiguous)
    const void* value_states;  // [B, Hkv, S_new, Ev]
    void* kcache;
    void* vcache;
    const int* block_table;    // [B, max_blocks]
    const int* seq_lengths;    // [B]
    long long ks_b, ks_h, ks_s, vs_b, vs_h, vs_s;
    int B, Hkv, S_new, E, Ev, block_size, max_blocks, num_blocks;
};

hipError_t launch_paged_attention(const PagedHeader& ph, int dtype, int E, int rb, hipStream_t stream);
hipError_t launch_paged_attention_wide(const PagedHeader& ph, int dtype, int E, hipStream_t stream);   // 128 rows per workgroup
hipError_t launch_copy_to_blocks(const CopyBlocksArgs& ca, int dtype, hipStream_t stream);

// ---- caller-side steps: input builder and fused key rotation + append ----
constexpr int MAX_POS_ENTRIES = 768;    // (fragment, worker) pairs per build_inputs launch
constexpr int MAX_APPEND_WORKERS = 64;  // workers per rope_append launch

struct BuildInputsArgs {
    int* locations;        // [F, W, S]
    float* cosines;        // [F, W, S, RotE]
    float* sines;
    const float* inv_freq; // [RotE / 2]
    float scaling;
    int F, W, S, RotE;
    // pos_end[f][w]: position one past the newest token of worker w, as seen through fragment f.  Either given ...
    int pos_end[MAX_POS_ENTRIES];
    // ... or, with len_dev, formed in the kernel from the fragment lengths in device memory: the table then holds
    // order[w][i] = the i-th fragment of worker w's order (W rows of F entries), and pos_end[f][w] is the sum of the
    // lengths of f and of everything behind it in that order.
    const int* len_dev;
};

struct AppendArgs {
    const void* k_src;     // [W, Hkv, S, E]  element strides ks_*, innermost contiguous
    const void* v_src;     // [W, Hkv, S, Ev]
    const void* cos;       // [W, S, RotE] element strides cs_w, cs_s (cs_s == 0 broadcasts one row over the tokens)
    const void* sin;
    long long ks_w, ks_h, ks_s, vs_w, vs_h, vs_s, cs_w, cs_s;
    int W, Hkv, S, E, Ev, RotE;
    void* k_dst[MAX_APPEND_WORKERS];     // segment buffers [Hkv, cap, E] / [Hkv, cap, Ev]
    void* v_dst[MAX_APPEND_WORKERS];
    int dst_len[MAX_APPEND_WORKERS];     // rows already in the segment; with len_dev: index into len_dev, whose entry
                                         // is the segment's length AFTER this append (rows already there = entry - n_new)
    int dst_cap[MAX_APPEND_WORKERS];
    int n_new[MAX_APPEND_WORKERS];       // the last n_new of the S source tokens are appended
    const int* len_dev;                  // segment lengths in device memory, or null
};

hipError_t launch_build_inputs(const BuildInputsArgs& a, int round_dtype, hipStream_t stream);
hipError_t launch_rope_append(const AppendArgs& a, int dtype, bool eager, bool cs16, hipStream_t stream);
// len_dev[f] += add[f] for f < F (F <= MAXF): the first node of a captured decode step
struct AdvanceArgs {
    int* len_dev;
    int F;
    int add[MAXF];
};
hipError_t launch_advance_lengths(const AdvanceArgs& a, hipStream_t stream);

}  // namespace hw
