// C ABI of the Hogwild! attention library: argument validation, split planning and launches.
// Validation and planning are pure host code and run before any HIP call, so they can be tested on a
// machine without a GPU.  No global mutable state apart from an immutable per-device CU-count cache.

#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstring>

#include "../../include/hogwild_hip.h"
#include "hogwild_kernels.h"
#include "hogwild_plan.h"

namespace {

using namespace hw::host;

constexpr int kMaxDevices = 64;
std::atomic<int> g_cus[kMaxDevices];   // 0 = not queried yet

int device_cus(int* cus) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return HW_ERR_NO_DEVICE;
    int c = g_cus[dev].load(std::memory_order_relaxed);
    if (c == 0) {
        e = hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev);
        if (e != hipSuccess) return (int)e;
        if (c <= 0) return HW_ERR_NO_DEVICE;
        g_cus[dev].store(c, std::memory_order_relaxed);
    }
    *cus = c;
    return HW_OK;
}

// Scratch of hw_fused_attention_static: the split-K partials (and, for rotary widths other than the head dimension,
// the rotated queries) of callers that cannot allocate.  One copy per GPU, held until the process ends.  On the host
// the array's name is only a handle: the device address comes from hipGetSymbolAddress, once per device.
__attribute__((used)) static __device__ __align__(256) unsigned char scratch[HW_STATIC_SCRATCH_BYTES];
std::atomic<void*> g_scratch[kMaxDevices];   // device address of `scratch` on each device; null = not asked yet

int static_scratch(void** ptr) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return HW_ERR_NO_DEVICE;
    void* p = g_scratch[dev].load(std::memory_order_acquire);
    if (p == nullptr) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return HW_ERR_NO_DEVICE;
        g_scratch[dev].store(p, std::memory_order_release);
    }
    *ptr = p;
    return HW_OK;
}

int run(const hw_problem* p, void* stream_, int fused, int stages = HW_STAGE_ATTENTION | HW_STAGE_MERGE) {
    int st = validate(p, fused);
    if (st != HW_OK) return st;
    int cus = 0;
    st = device_cus(&cus);
    if (st != HW_OK) return st;
    CallPlan cp;
    st = plan_call(p, cus, &cp, fused);
    if (st != HW_OK) return st;
    if (p->workspace == nullptr || p->workspace_bytes < cp.workspace_bytes || !aligned16(p->workspace)) return HW_ERR_WORKSPACE;
    const hw_plan& plan0 = cp.plan[0];
    // the VALU logits exist for what they are measured on: the fused entry with full rotary width, one row block, host lengths
    if (p->variant == HW_VARIANT_VALU_QK && (!fused || p->RotE != p->E || plan0.row_blocks != 1 || p->len_dev != nullptr)) return HW_ERR_UNSUPPORTED;

    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    const size_t esz = elem_size(p->dtype);
    const char* q_in = reinterpret_cast<const char*>(p->q);
    bool prerotated = !fused;
    if (fused && p->RotE != p->E) {
        void* rqbuf = p->rq;
        if (rqbuf == nullptr) rqbuf = reinterpret_cast<char*>(p->workspace) + cp.partial_bytes;
        if (stages & HW_STAGE_ATTENTION) {
            hipError_t er = hw::launch_rope(rqbuf, p->q, p->cosines, p->sines, p->dtype, p->F, p->W, p->Hq, p->S, p->E, p->RotE, stream);
            if (er != hipSuccess) return (int)er;
        }
        q_in = reinterpret_cast<const char*>(rqbuf);
        prerotated = true;
    }
    const int rows = plan0.rows;
    float* const part_o = reinterpret_cast<float*>(p->workspace);
    float* const part_ml = part_o + (size_t)p->Hkv * cp.slots * rows * p->Ev;
    // One workgroup per kv head and row group holds whole rows: it writes out / lse itself and the merge launch is
    // dropped (the 128-row kernel has an epilogue of its own and always goes through the merge).
    const bool direct = cp.groups == 1 && plan0.wgs_per_head == 1 && stages == (HW_STAGE_ATTENTION | HW_STAGE_MERGE) &&
                        plan0.row_blocks != hw::WIDE_ROW_BLOCKS;
    auto magic = [](int d) { return magic_of(d); };

    hipError_t e = hipSuccess;
    for (int gi = 0; gi < cp.groups && (stages & HW_STAGE_ATTENTION); ++gi) {
        const hw_plan& plan = cp.plan[gi];
        const int f0 = cp.first[gi], nf = cp.count[gi];
        const size_t ws_rows = (size_t)p->W * p->S;                    // (worker, token) pairs per fragment
        const size_t q_frag = ws_rows * p->Hq * p->E * esz;            // bytes of one fragment's rotated queries
        hw::KernelArgs ka;
        std::memset(&ka, 0, sizeof(ka));
        for (int f = 0; f < nf; ++f) {
            ka.frag.k[f] = p->k[f0 + f];
            ka.frag.v[f] = p->v[f0 + f];
            ka.frag.lc[f].len = p->len[f0 + f];
            ka.frag.lc[f].cap = p->cap != nullptr ? p->cap[f0 + f] : p->len[f0 + f];
        }
        for (int f = 0; f <= HW_MAX_LAUNCH_FRAGMENTS; ++f) ka.frag.tile_begin[f] = plan.tile_begin[f];
        for (int i = 0; i <= HW_MAX_SPLITS; ++i) ka.wg_tile[i] = plan.wg_tile_begin[i];
        // everything indexed by fragment starts at this group's first fragment
        ka.h.q = prerotated ? q_in + (size_t)f0 * q_frag : q_in;
        ka.h.loc = p->locations + (size_t)f0 * ws_rows;
        ka.h.cos = p->cosines != nullptr ? p->cosines + (size_t)f0 * ws_rows * p->RotE : nullptr;
        ka.h.sin = p->sines != nullptr ? p->sines + (size_t)f0 * ws_rows * p->RotE : nullptr;
        ka.h.rq = (fused && !prerotated && p->rq != nullptr) ? reinterpret_cast<char*>(p->rq) + (size_t)f0 * q_frag : nullptr;
        ka.h.part_o = part_o + (size_t)cp.slot_base[gi] * rows * p->Ev;
        ka.h.part_ml = part_ml + (size_t)cp.slot_base[gi] * rows * 2;
        ka.h.len_dev = p->len_dev;
        ka.h.F = nf; ka.h.W = p->W; ka.h.Hq = p->Hq; ka.h.Hkv = p->Hkv; ka.h.S = p->S;
        ka.h.R = rows;
        ka.h.nrg = plan.row_groups;
        ka.h.wgs_per_head = plan.wgs_per_head;
        ka.h.nwg = plan.workgroups;
        ka.h.slot_stride = cp.slots;
        ka.h.flags = ((plan.workgroups % 8 == 0) ? hw::KH_XCD_REMAP : 0) | (direct ? hw::KH_DIRECT : 0) | (prerotated ? hw::KH_PREROTATED : 0);
        if (direct) {
            ka.h.part_o = reinterpret_cast<float*>(p->out);
            ka.h.part_ml = p->lse;
        }
        ka.h.sc = (float)((double)p->scale * 1.4426950408889634074);
        // multipliers for the in-kernel divisions (exact for numerators < 2^20 and divisors < 2^12, both validated)
        ka.h.magic_gq = magic(p->Hq / p->Hkv);
        ka.h.magic_s = magic(p->S);
        ka.h.magic_nrg = magic(plan.row_groups);
        ka.h.magic_wg = magic(plan.wgs_per_head);
        if (plan.row_blocks == hw::WIDE_ROW_BLOCKS)
            e = hw::launch_attention_wide(ka, p->dtype, p->E, stream);
        else
            e = hw::launch_attention(ka, p->dtype, p->E, plan.row_blocks, p->variant, stream);
        if (e != hipSuccess) return (int)e;
    }
    if (!(stages & HW_STAGE_MERGE) || direct) return (int)e;
    hw::MergeArgs ma;
    ma.part_o = part_o;
    ma.part_ml = part_ml;
    ma.out = p->out;
    ma.lse = p->lse;
    ma.W = p->W; ma.Hq = p->Hq; ma.Hkv = p->Hkv; ma.S = p->S; ma.R = rows;
    ma.wgs_per_head = cp.slots;
    ma.xcd_local = (cp.groups == 1 && plan0.workgroups % 8 == 0 && p->Hkv % 8 == 0) ? 1 : 0;
    ma.row_tab = nullptr;
    ma.pslots = 0;
    e = hw::launch_merge(ma, p->dtype, p->Ev, stream);
    return (int)e;
}

// ---------------------------------------------------------------------------------------------------------
// paged variants
// ---------------------------------------------------------------------------------------------------------
int paged_run(const hw_paged_problem* p, void* stream_, int stages) {
    int st = paged_validate(p);
    if (st != HW_OK) return st;
    int cus = 0;
    st = device_cus(&cus);
    if (st != HW_OK) return st;
    hw_paged_plan plan;
    st = paged_plan(p, cus, &plan);
    if (st != HW_OK) return st;
    if (plan.rows == 0) return HW_OK;       // no query tokens
    if (p->workspace == nullptr || p->workspace_bytes < plan.workspace_bytes || !aligned16(p->workspace)) return HW_ERR_WORKSPACE;
    hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
    const bool varlen = p->cu_seqlens_q != nullptr;
    auto magic = [](int d) { return magic_of(d); };

    hw::PagedHeader ph;
    std::memset(&ph, 0, sizeof(ph));
    ph.q = p->q;
    ph.loc = p->locations;
    ph.frag_len = p->fragment_lengths;
    ph.kcache = p->key_cache;
    ph.vcache = p->value_cache;
    ph.block_table = p->block_table;
    ph.cu_q = p->cu_seqlens_q;
    // partial sums by (split, row), or -- planned on the device -- by workgroup slot, then the merge's row table
    const bool planned = plan.device_planned != 0;
    const size_t prows = planned ? (size_t)plan.row_groups * hw::PLAN_SLOT_ROWS : (size_t)plan.splits * plan.rows;
    ph.part_o = reinterpret_cast<float*>(p->workspace);
    ph.part_ml = ph.part_o + (size_t)p->Hkv * prows * p->Ev;
    int* row_tab = reinterpret_cast<int*>(ph.part_ml + (size_t)p->Hkv * prows * 2);
    ph.F = p->F; ph.W = p->W; ph.Hq = p->Hq; ph.Hkv = p->Hkv;
    ph.LW = varlen ? p->total_q : p->W;
    ph.LS = varlen ? 1 : p->S;
    ph.R = plan.rows;
    ph.block_size = p->block_size; ph.max_blocks = p->max_blocks; ph.num_blocks = p->num_blocks;
    ph.nsplit = plan.splits;
    ph.nitems = plan.row_groups;
    ph.nrg = varlen ? 1 : plan.row_groups / p->W;
    ph.nwg = plan.workgroups;
    ph.flags = ((plan.workgroups % 8 == 0) ? hw::PH_XCD_REMAP : 0) | (planned ? hw::PH_PLANNED : 0);
    ph.sc = (float)((double)p->scale * 1.4426950408889634074);
    ph.magic_gq = magic(p->Hq / p->Hkv);
    ph.magic_ls = magic(ph.LS);
    ph.magic_bs = magic(p->block_size);
    ph.magic_nsplit = magic(ph.nsplit);
    ph.magic_nitems = magic(ph.nitems);
    ph.magic_nrg = magic(ph.nrg);

    hipError_t e = hipSuccess;
    if (stages & HW_STAGE_ATTENTION) {
        if (plan.row_blocks == hw::WIDE_ROW_BLOCKS) e = hw::launch_paged_attention_wide(ph, p->dtype, p->E, stream);
        else e = hw::launch_paged_attention(ph, p->dtype, p->E, plan.row_blocks, stream);
        if (e != hipSuccess) return (int)e;
    }
    if (!(stages & HW_STAGE_MERGE)) return (int)e;
    hw::MergeArgs ma;
    ma.part_o = ph.part_o;
    ma.part_ml = ph.part_ml;
    ma.out = p->out;
    ma.lse = p->lse;
    ma.W = ph.LW; ma.Hq = p->Hq; ma.Hkv = p->Hkv; ma.S = ph.LS; ma.R = plan.rows;
    ma.wgs_per_head = plan.splits;
    // a variable-length launch may leave row groups of the grid unused, and with them parts of an XCD's share
    // (a launch planned on the device keeps every slot of a kv head on the head's XCD whatever the slots do)
    ma.xcd_local = ((!varlen || planned) && plan.workgroups % 8 == 0 && p->Hkv % 8 == 0) ? 1 : 0;
    ma.row_tab = planned ? row_tab : nullptr;
    ma.pslots = planned ? plan.row_groups : 0;
    if (planned) ma.wgs_per_head = 8;       // a row's slots are device data: the merge shape that suits a handful of them
    e = hw::launch_merge(ma, p->dtype, p->Ev, stream);
    return (int)e;
}

int copy_blocks_run(const hw_copy_blocks* c, void* stream) {
    if (c == nullptr) return HW_ERR_NULL;
    if (c->dtype != HW_F32 && c->dtype != HW_F16 && c->dtype != HW_BF16) return HW_ERR_DTYPE;
    if (c->B < 0 || c->Hkv < 1 || c->S_new < 0 || c->E < 1 || c->Ev < 1) return HW_ERR_SHAPE;
    if (c->block_size < 1 || c->max_blocks < 1 || c->num_blocks < 1) return HW_ERR_SHAPE;
    if ((long long)c->num_blocks * c->Hkv * c->block_size >= (1ll << 31)) return HW_ERR_SHAPE;
    if (c->B == 0 || c->S_new == 0) return HW_OK;
    if (c->key_states == nullptr || c->value_states == nullptr || c->key_cache == nullptr || c->value_cache == nullptr ||
        c->block_table == nullptr || c->seq_lengths == nullptr)
        return HW_ERR_NULL;
    hw::CopyBlocksArgs a;
    a.key_states = c->key_states; a.value_states = c->value_states;
    a.kcache = c->key_cache; a.vcache = c->value_cache;
    a.block_table = c->block_table; a.seq_lengths = c->seq_lengths;
    a.ks_b = c->ks_b; a.ks_h = c->ks_h; a.ks_s = c->ks_s; a.vs_b = c->vs_b; a.vs_h = c->vs_h; a.vs_s = c->vs_s;
    a.B = c->B; a.Hkv = c->Hkv; a.S_new = c->S_new; a.E = c->E; a.Ev = c->Ev;
    a.block_size = c->block_size; a.max_blocks = c->max_blocks; a.num_blocks = c->num_blocks;
    return (int)hw::launch_copy_to_blocks(a, c->dtype, reinterpret_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------------------------------------------------------
// caller-side steps
// ---------------------------------------------------------------------------------------------------------
int build_inputs_run(int32_t* locations, float* cosines, float* sines, const int32_t* pos_end, const float* inv_freq,
                     float scaling, int round_dtype, int F, int W, int S, int RotE, void* stream) {
    if (F < 1 || W < 1 || S < 1 || RotE < 0 || (RotE & 1)) return HW_ERR_SHAPE;
    if (round_dtype != HW_F32 && round_dtype != HW_F16 && round_dtype != HW_BF16) return HW_ERR_DTYPE;
    if (locations == nullptr || pos_end == nullptr) return HW_ERR_NULL;
    if (RotE > 0 && (cosines == nullptr || sines == nullptr || inv_freq == nullptr)) return HW_ERR_NULL;
    if (W > hw::MAX_POS_ENTRIES) return HW_ERR_UNSUPPORTED;
    if ((long long)F * W * S * (RotE > 0 ? RotE : 1) >= (1ll << 31)) return HW_ERR_SHAPE;
    const int fchunk = hw::MAX_POS_ENTRIES / W;      // fragments per launch
    for (int f0 = 0; f0 < F; f0 += fchunk) {
        const int nf = F - f0 < fchunk ? F - f0 : fchunk;
        hw::BuildInputsArgs a;
        a.locations = locations + (size_t)f0 * W * S;
        a.cosines = RotE > 0 ? cosines + (size_t)f0 * W * S * RotE : nullptr;
        a.sines = RotE > 0 ? sines + (size_t)f0 * W * S * RotE : nullptr;
        a.inv_freq = inv_freq;
        a.scaling = scaling;
        a.F = nf; a.W = W; a.S = S; a.RotE = RotE;
        a.len_dev = nullptr;
        std::memcpy(a.pos_end, pos_end + (size_t)f0 * W, sizeof(int) * (size_t)nf * W);
        hipError_t e = hw::launch_build_inputs(a, round_dtype, reinterpret_cast<hipStream_t>(stream));
        if (e != hipSuccess) return (int)e;
    }
    return HW_OK;
}

int build_inputs_dev_run(int32_t* locations, float* cosines, float* sines, const int32_t* len_dev, const int32_t* orders,
                         const float* inv_freq, float scaling, int round_dtype, int F, int W, int S, int RotE, void* stream) {
    if (F < 1 || F > HW_MAX_LAUNCH_FRAGMENTS || W < 1 || S < 1 || RotE < 0 || (RotE & 1)) return HW_ERR_SHAPE;
    if (round_dtype != HW_F32 && round_dtype != HW_F16 && round_dtype != HW_BF16) return HW_ERR_DTYPE;
    if (locations == nullptr || len_dev == nullptr || orders == nullptr) return HW_ERR_NULL;
    if (RotE > 0 && (cosines == nullptr || sines == nullptr || inv_freq == nullptr)) return HW_ERR_NULL;
    if ((long long)F * W > hw::MAX_POS_ENTRIES) return HW_ERR_UNSUPPORTED;
    if ((long long)F * W * S * (RotE > 0 ? RotE : 1) >= (1ll << 31)) return HW_ERR_SHAPE;
    for (int w = 0; w < W; ++w) {      // every worker's order is a permutation of the fragments
        unsigned long long seen = 0;
        for (int i = 0; i < F; ++i) {
            const int g = orders[(size_t)w * F + i];
            if (g < 0 || g >= F || (seen >> g & 1ull)) return HW_ERR_SHAPE;
            seen |= 1ull << g;
        }
    }
    hw::BuildInputsArgs a;
    a.locations = locations;
    a.cosines = RotE > 0 ? cosines : nullptr;
    a.sines = RotE > 0 ? sines : nullptr;
    a.inv_freq = inv_freq;
    a.scaling = scaling;
    a.F = F; a.W = W; a.S = S; a.RotE = RotE;
    a.len_dev = len_dev;
    std::memcpy(a.pos_end, orders, sizeof(int) * (size_t)F * W);
    return (int)hw::launch_build_inputs(a, round_dtype, reinterpret_cast<hipStream_t>(stream));
}

int advance_lengths_run(int32_t* len_dev, const int32_t* add, int F, void* stream) {
    if (len_dev == nullptr || add == nullptr) return HW_ERR_NULL;
    if (F < 1 || F > HW_MAX_LAUNCH_FRAGMENTS) return HW_ERR_FRAGMENTS;
    hw::AdvanceArgs a;
    std::memset(&a, 0, sizeof(a));
    a.len_dev = len_dev;
    a.F = F;
    for (int f = 0; f < F; ++f) a.add[f] = add[f];
    return (int)hw::launch_advance_lengths(a, reinterpret_cast<hipStream_t>(stream));
}

int rope_append_run(const hw_append* p, void* stream) {
    if (p == nullptr) return HW_ERR_NULL;
    if (p->dtype != HW_F32 && p->dtype != HW_F16 && p->dtype != HW_BF16) return HW_ERR_DTYPE;
    if (p->cs_dtype != HW_F32 && p->cs_dtype != p->dtype) return HW_ERR_DTYPE;
    if (p->mode != HW_ROPE_EAGER && p->mode != HW_ROPE_FUSED) return HW_ERR_SHAPE;
    if (p->W < 1 || p->Hkv < 1 || p->S < 0 || p->E < 1 || p->Ev < 1) return HW_ERR_SHAPE;
    if (p->RotE < 0 || p->RotE > p->E || (p->RotE & 1)) return HW_ERR_SHAPE;
    if (p->k_dst == nullptr || p->v_dst == nullptr || p->dst_len == nullptr || p->dst_cap == nullptr || p->n_new == nullptr) return HW_ERR_NULL;
    bool any = false;
    for (int w = 0; w < p->W; ++w) {
        if (p->n_new[w] < 0 || p->n_new[w] > p->S || p->dst_len[w] < 0) return HW_ERR_SHAPE;
        // (with the lengths in device memory dst_len is an index and the kernel itself drops what does not fit)
        if (p->len_dev == nullptr && (long long)p->dst_len[w] + p->n_new[w] > p->dst_cap[w]) return HW_ERR_SHAPE;    // the segment is full
        if (p->n_new[w] > 0) {
            if (p->k_dst[w] == nullptr || p->v_dst[w] == nullptr) return HW_ERR_NULL;
            any = true;
        }
    }
    if (!any) return HW_OK;
    if (p->key_states == nullptr || p->value_states == nullptr) return HW_ERR_NULL;
    if (p->RotE > 0 && (p->cosines == nullptr || p->sines == nullptr)) return HW_ERR_NULL;
    for (int w0 = 0; w0 < p->W; w0 += hw::MAX_APPEND_WORKERS) {
        const int nw = p->W - w0 < hw::MAX_APPEND_WORKERS ? p->W - w0 : hw::MAX_APPEND_WORKERS;
        const size_t sz = elem_size(p->dtype), csz = p->cs_dtype == HW_F32 ? 4 : 2;
        hw::AppendArgs a;
        std::memset(&a, 0, sizeof(a));
        a.k_src = reinterpret_cast<const char*>(p->key_states) + (long long)w0 * p->ks_w * (long long)sz;
        a.v_src = reinterpret_cast<const char*>(p->value_states) + (long long)w0 * p->vs_w * (long long)sz;
        a.cos = p->RotE > 0 ? reinterpret_cast<const char*>(p->cosines) + (long long)w0 * p->cs_w * (long long)csz : nullptr;
        a.sin = p->RotE > 0 ? reinterpret_cast<const char*>(p->sines) + (long long)w0 * p->cs_w * (long long)csz : nullptr;
        a.ks_w = p->ks_w; a.ks_h = p->ks_h; a.ks_s = p->ks_s;
        a.vs_w = p->vs_w; a.vs_h = p->vs_h; a.vs_s = p->vs_s;
        a.cs_w = p->cs_w; a.cs_s = p->cs_s;
        a.W = nw; a.Hkv = p->Hkv; a.S = p->S; a.E = p->E; a.Ev = p->Ev; a.RotE = p->RotE;
        for (int w = 0; w < nw; ++w) {
            a.k_dst[w] = p->k_dst[w0 + w];
            a.v_dst[w] = p->v_dst[w0 + w];
            a.dst_len[w] = p->dst_len[w0 + w];
            a.dst_cap[w] = p->dst_cap[w0 + w];
            a.n_new[w] = p->n_new[w0 + w];
        }
        a.len_dev = p->len_dev;
        hipError_t e = hw::launch_rope_append(a, p->dtype, p->mode == HW_ROPE_EAGER, p->cs_dtype != HW_F32, reinterpret_cast<hipStream_t>(stream));
        if (e != hipSuccess) return (int)e;
    }
    return HW_OK;
}

}  // namespace

extern "C" {

int hw_version(void) { return HW_ABI_VERSION; }

const char* hw_status_string(int status) {
    switch (status) {
        case HW_OK: return "ok";
        case HW_ERR_NULL: return "required pointer is NULL";
        case HW_ERR_DTYPE: return "unknown dtype";
        case HW_ERR_SHAPE: return "invalid or inconsistent shape";
        case HW_ERR_UNSUPPORTED: return "no kernel instantiated for this shape (need E == Ev in {64, 128})";
        case HW_ERR_FRAGMENTS: return "fragment count out of range";
        case HW_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case HW_ERR_ALIGN: return "device pointer not 16-byte aligned";
        case HW_ERR_NO_DEVICE: return "no usable HIP device";
        case HW_ERR_STATIC_SCRATCH: return "problem needs more scratch than HW_STATIC_SCRATCH_BYTES (use hw_fused_attention with a caller workspace)";
        default: break;
    }
    if (status > 0) return hipGetErrorString(static_cast<hipError_t>(status));
    return "unknown status";
}

int hw_validate(const hw_problem* p, int fused) { return validate(p, fused); }

int hw_plan_debug(const hw_problem* p, int num_cus, hw_plan* plan) {
    // planning needs only the shape and the lengths
    if (p == nullptr || plan == nullptr || p->len == nullptr) return HW_ERR_NULL;
    if (p->F < 1 || p->F > HW_MAX_LAUNCH_FRAGMENTS) return HW_ERR_FRAGMENTS;
    if (p->W < 1 || p->Hq < 1 || p->Hkv < 1 || p->S < 1 || p->Ev < 1 || p->Hq % p->Hkv != 0) return HW_ERR_SHAPE;
    for (int f = 0; f < p->F; ++f)
        if (p->len[f] < 0) return HW_ERR_SHAPE;
    return make_plan(p, num_cus, plan);
}

static int workspace_bytes_for(const hw_problem* p, int fused, size_t* bytes) {
    if (bytes == nullptr) return HW_ERR_NULL;
    if (p == nullptr || p->len == nullptr) return HW_ERR_NULL;
    int cus = 0;
    int st = device_cus(&cus);
    if (st != HW_OK) return st;
    CallPlan cp;
    st = plan_call(p, cus, &cp, fused);
    if (st != HW_OK) return st;
    *bytes = cp.workspace_bytes;
    return HW_OK;
}

int hw_workspace_bytes(const hw_problem* p, size_t* bytes) { return workspace_bytes_for(p, 1, bytes); }

int hw_sdpa_workspace_bytes(const hw_problem* p, size_t* bytes) { return workspace_bytes_for(p, 0, bytes); }

int hw_fused_attention(const hw_problem* p, void* stream) { return run(p, stream, 1); }

int hw_sdpa(const hw_problem* p, void* stream) { return run(p, stream, 0); }

int hw_fused_attention_static(const hw_problem* p, void* stream) {
    int st = validate(p, 1);
    if (st != HW_OK) return st;
    int cus = 0;
    st = device_cus(&cus);
    if (st != HW_OK) return st;
    CallPlan cp;
    hw_problem q = *p;
    st = plan_call(&q, cus, &cp, 1);
    if (st != HW_OK) return st;
    if (cp.workspace_bytes > (size_t)HW_STATIC_SCRATCH_BYTES && p->row_blocks == 0 && cp.plan[0].row_blocks == hw::WIDE_ROW_BLOCKS) {
        // the 128-row workgroups write a partial per split for all rows of a kv head: the 32-row kernel needs a quarter
        // of that with its fewer splits per row group, and the caller left the choice to the library
        q.row_blocks = 2;
        st = plan_call(&q, cus, &cp, 1);
        if (st != HW_OK) return st;
    }
    if (cp.workspace_bytes > (size_t)HW_STATIC_SCRATCH_BYTES) return HW_ERR_STATIC_SCRATCH;
    void* ptr = nullptr;
    st = static_scratch(&ptr);
    if (st != HW_OK) return st;
    q.workspace = ptr;
    q.workspace_bytes = (size_t)HW_STATIC_SCRATCH_BYTES;
    return run(&q, stream, 1);
}

int hw_fused_attention_stages(const hw_problem* p, void* stream, int stages) {
    if ((stages & (HW_STAGE_ATTENTION | HW_STAGE_MERGE)) == 0 || (stages & ~(HW_STAGE_ATTENTION | HW_STAGE_MERGE)) != 0) return HW_ERR_SHAPE;
    return run(p, stream, 1, stages);
}

int hw_rope(void* out, const void* q, const float* cosines, const float* sines, int dtype, int F, int W, int Hq, int S, int E,
            int RotE, void* stream) {
    if (out == nullptr || q == nullptr) return HW_ERR_NULL;
    if (dtype != HW_F32 && dtype != HW_F16 && dtype != HW_BF16) return HW_ERR_DTYPE;
    if (F < 1 || W < 1 || Hq < 1 || S < 1 || E < 1) return HW_ERR_SHAPE;
    if (RotE < 0 || RotE > E || (RotE & 1)) return HW_ERR_SHAPE;
    if (RotE > 0 && (cosines == nullptr || sines == nullptr)) return HW_ERR_NULL;
    return (int)hw::launch_rope(out, q, cosines, sines, dtype, F, W, Hq, S, E, RotE, reinterpret_cast<hipStream_t>(stream));
}

int hw_paged_validate(const hw_paged_problem* p) { return paged_validate(p); }

int hw_paged_plan_debug(const hw_paged_problem* p, int num_cus, hw_paged_plan* plan) {
    if (p == nullptr || plan == nullptr) return HW_ERR_NULL;
    if (p->W < 1 || p->Hq < 1 || p->Hkv < 1 || p->Ev < 1 || p->Hq % p->Hkv != 0 || p->block_size < 1 || p->max_blocks < 1) return HW_ERR_SHAPE;
    if (p->cu_seqlens_q != nullptr ? p->total_q < 0 : p->S < 1) return HW_ERR_SHAPE;
    return paged_plan(p, num_cus, plan);
}

int hw_paged_workspace_bytes(const hw_paged_problem* p, size_t* bytes) {
    if (bytes == nullptr) return HW_ERR_NULL;
    int cus = 0;
    int st = device_cus(&cus);
    if (st != HW_OK) return st;
    hw_paged_plan plan;
    st = hw_paged_plan_debug(p, cus, &plan);
    if (st != HW_OK) return st;
    *bytes = plan.workspace_bytes;
    return HW_OK;
}

int hw_paged_sdpa(const hw_paged_problem* p, void* stream) {
    if (p != nullptr && p->cu_seqlens_q != nullptr) return HW_ERR_SHAPE;
    return paged_run(p, stream, HW_STAGE_ATTENTION | HW_STAGE_MERGE);
}

int hw_varlen_paged_sdpa(const hw_paged_problem* p, void* stream) {
    if (p != nullptr && p->cu_seqlens_q == nullptr) return HW_ERR_NULL;
    return paged_run(p, stream, HW_STAGE_ATTENTION | HW_STAGE_MERGE);
}

int hw_paged_sdpa_stages(const hw_paged_problem* p, void* stream, int stages) {
    if ((stages & (HW_STAGE_ATTENTION | HW_STAGE_MERGE)) == 0 || (stages & ~(HW_STAGE_ATTENTION | HW_STAGE_MERGE)) != 0) return HW_ERR_SHAPE;
    return paged_run(p, stream, stages);
}

int hw_copy_to_blocks(const hw_copy_blocks* c, void* stream) { return copy_blocks_run(c, stream); }

int hw_build_inputs(int32_t* locations, float* cosines, float* sines, const int32_t* pos_end, const float* inv_freq,
                    float attention_scaling, int round_dtype, int F, int W, int S, int RotE, void* stream) {
    return build_inputs_run(locations, cosines, sines, pos_end, inv_freq, attention_scaling, round_dtype, F, W, S, RotE, stream);
}

int hw_build_inputs_dev(int32_t* locations, float* cosines, float* sines, const int32_t* len_dev, const int32_t* orders,
                        const float* inv_freq, float attention_scaling, int round_dtype, int F, int W, int S, int RotE,
                        void* stream) {
    return build_inputs_dev_run(locations, cosines, sines, len_dev, orders, inv_freq, attention_scaling, round_dtype, F, W, S, RotE,
                                stream);
}

int hw_advance_lengths(int32_t* len_dev, const int32_t* add, int F, void* stream) { return advance_lengths_run(len_dev, add, F, stream); }

int hw_rope_append(const hw_append* a, void* stream) { return rope_append_run(a, stream); }

int hw_device_cus(void) {
    int c = 0;
    return device_cus(&c) == HW_OK ? c : 0;
}

}  // extern "C"
