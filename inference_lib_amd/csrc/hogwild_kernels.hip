// Hogwild! fragmented-KV decode attention for gfx950 (MI355X, CDNA4, wave64).
//
// One workgroup = one kv head x one contiguous range of 32-token tiles (crossing fragment boundaries)
// x up to 32 query rows, where a "row" is one (worker, token, q-head-in-group) triple (more than 96 rows per
// kv head: attention_wide_kernel, hogwild_wide.hip).  All rows that
// share a kv head are multiplied against each K/V tile once, so KV is read from HBM once per step
// instead of once per (worker, token) as in the reference (src/kernels/kernel_v21.cuh:62-66).
//
// Per wave and tile:
//   S^T[token, row] = K[token, :] . Q[row, :]        v_mfma_f32_16x16x32 (bf16/f16) or 16x16x4 (f32)
//   online softmax in base 2 on the accumulator layout (rows live on lane%16, so every per-row scalar
//   is lane-local; only the row max needs two cross-lane steps)
//   O^T[ev, row] += V^T[ev, token] . P^T[token, row]
// K goes global -> LDS by direct transfers (no VGPR staging) into a per-wave staging slot, XOR-swizzled so that
// the A-operand reads (lane = token, 16 B of the head dim) are free of bank conflicts;
// V is loaded as whole 256-byte rows (16 lanes x 16 B) and transposed in registers with v_perm_b32,
// using the freedom to permute the reduced (token) index identically in both MFMA operands.
// The query is rotated per fragment in the prologue (src/rope.cuh:18-51), rounded to the storage type
// like the reference's `rq` scratch (src/rope.cuh:43-45) and kept in registers as the B operand.
//
// Partials (unnormalised O, running max, sum) go to the workspace; a second kernel merges them by
// log-sum-exp (the role of src/kernels/kernel_v21.cuh:605-656) and writes out + lse.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/hogwild_hip.h"
#include "hogwild_kernels.h"

namespace hw {

// Phase timestamps for kernel tuning; compiled in only with -DHW_CLOCKS (never in the shipped library).
#ifdef HW_CLOCKS
__device__ unsigned long long hw_clock_buf[4096 * 16];
#define HW_MARK(i)                                                                                  \
    do {                                                                                            \
        if ((threadIdx.x & 63) == 0 && blockIdx.x < 1024)                                           \
            hw_clock_buf[(blockIdx.x * 4 + (threadIdx.x >> 6)) * 16 + (i)] = wall_clock64();         \
    } while (0)
#else
#define HW_MARK(i) do { } while (0)
#endif

}  // namespace hw

#include "hogwild_device.h"

namespace hw {

// MINW = waves per SIMD the register budget is sized for: 2 (<= 256 VGPRs) when one 16-row block is live,
// 1 (<= 512 VGPRs) when two row blocks or fp32 operands make the tile registers too large.
// PF = tiles a wave keeps in flight.  PRE = queries arrive rotated (hogwild_sdpa), else fused rotation.
// VS = logits by VALU dot products instead of MFMA (one row block only): the alternative the MFMA choice is measured against.
// DEVLEN = the current fragment lengths come from device memory (header.len_dev); the lengths in the table are then
// the bounds the split was planned for, and a captured launch stays valid while the segments grow up to them.
template <class DT, int E, int EV, int RB, int MINW, int PF, bool PRE, bool DEVLEN = false, bool VS = false>
__global__ __launch_bounds__(NTHREADS, MINW) void attention_kernel(const KernelArgs args) {
    typedef Geo<DT, E, EV> G;
    constexpr int ROWS = RB * 16;

    typedef hw::Exchange<ROWS, EV> Ex;
    constexpr int SBYTES = NWAVES * G::KSTAGE;
    // With one wave per SIMD there are registers to spare: the query operands of a segment stay in them (QREG).  The fp32
    // kernel with one row block goes further (LANEROT): every wave loads and rotates its own operands in those registers,
    // no copy of the rotated rows in LDS and no barrier in the prologue of a segment (config 1: 7.35 -> 7.1 us).  With
    // two row blocks of 16-bit queries the 26 loads per wave this takes, against 7, cost more than the barriers did.
    constexpr bool QREG = MINW == 1;
    constexpr bool LANEROT = QREG && !VS && G::SZ == 4 && RB == 1;
    __shared__ __attribute__((aligned(16))) char q_lds[LANEROT ? 16 : ROWS * G::QSTR];
    __shared__ int lim_lds[LANEROT ? 1 : ROWS];
    // One K staging slot per tile in flight, each a separate LDS object so that the wait for a slot's incoming
    // transfers does not extend to the other slots.  Kernels that run one workgroup per CU have LDS to spare and give
    // the epilogue exchange memory of its own, so that a wave can hand over its accumulators the moment it is done; in
    // the others the exchange reuses the memory of slot 0.
    constexpr bool EXSEP = MINW == 1 && sizeof(Ex) + PF * SBYTES + (LANEROT ? 0 : ROWS * G::QSTR) + 1024 <= 160 * 1024;
    union Slot0 {
        char k[SBYTES];
        char ex[EXSEP ? 16 : sizeof(Ex)];
    };
    __shared__ __attribute__((aligned(16))) Slot0 slot0;
    __shared__ __attribute__((aligned(16))) char slot1[PF > 1 ? SBYTES : 16];
    __shared__ __attribute__((aligned(16))) char slot2[PF > 2 ? SBYTES : 16];
    __shared__ __attribute__((aligned(16))) char ex_own[EXSEP ? sizeof(Ex) : 16];
    Ex& ex = *reinterpret_cast<Ex*>(EXSEP ? ex_own : slot0.ex);
    static_assert(PF <= 3, "three staging slots");

    const int tid = threadIdx.x;
    HW_MARK(8);
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int q = lane >> 4;
    char* const kslots[3] = {slot0.k + wv * G::KSTAGE, slot1 + (PF > 1 ? wv * G::KSTAGE : 0), slot2 + (PF > 2 ? wv * G::KSTAGE : 0)};
    // Everything the kernel needs from its arguments is requested here in one burst, before anything waits:
    // the fragment table and the workgroup boundary table with one vector load per lane and array, the 32
    // scalar dwords with two 64-byte scalar loads.  The argument segment is slow to reach and the compiler
    // would otherwise fetch it lazily, one dependent round trip after another.  The setup that does not depend
    // on the arguments runs while they are in flight.
    const int fl = lane & (MAXF - 1);
    const unsigned long long my_k = reinterpret_cast<unsigned long long>(args.frag.k[fl]);
    const unsigned long long my_v = reinterpret_cast<unsigned long long>(args.frag.v[fl]);
    const FragTable::LenCap my_lc = args.frag.lc[fl];
    int my_len = my_lc.len;
    const int my_cap = my_lc.cap;
    const int my_tb = args.frag.tile_begin[fl];
    const int my_te = args.frag.tile_begin[fl + 1];
    int my_wt[MAX_SPLITS / 64], my_wt1[MAX_SPLITS / 64];
#pragma unroll
    for (int i = 0; i < MAX_SPLITS / 64; ++i) {
        my_wt[i] = args.wg_tile[lane + 64 * i];
        my_wt1[i] = args.wg_tile[lane + 64 * i + 1];
    }
    typedef int i32x16 __attribute__((ext_vector_type(16)));
    struct HeaderBits { i32x16 lo, hi; };
    HeaderBits hb;
    {
        const auto argp = __builtin_amdgcn_kernarg_segment_ptr();
        asm volatile("s_load_dwordx16 %0, %2, 0x0\n\ts_load_dwordx16 %1, %2, 0x40" : "=&s"(hb.lo), "=&s"(hb.hi) : "s"(argp) : "memory");
    }
    unsigned koff[G::KL];
    k_lane_offsets<G>(koff, lane);
    WaveState<RB, G::NOC> st;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        st.m[rb] = NEG_BIG;
        st.l[rb] = 0.f;
#pragma unroll
        for (int c = 0; c < G::NOC; ++c) st.o[rb][c] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    st.fresh = true;
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(hb.lo), "+s"(hb.hi) : : "memory");   // the header is usable from here on
    const DevHeader a = __builtin_bit_cast(DevHeader, hb);
    if constexpr (DEVLEN) my_len = min(my_len, a.len_dev[fl < a.F ? fl : 0]);

    // consecutive logical ids stay on one XCD (hardware deals workgroups round-robin over the 8 XCDs)
    int bid = blockIdx.x;
    if (a.flags & KH_XCD_REMAP) bid = (bid & 7) * (a.nwg >> 3) + (bid >> 3);
    const int hg = fast_div(bid, a.magic_nrg);            // (kv head, split) pair
    const int rg = bid - hg * a.nrg;
    const int hkv = fast_div(hg, a.magic_wg);
    const int g = hg - hkv * a.wgs_per_head;

    int T0 = 0, T1 = 0;
#pragma unroll
    for (int i = 0; i < MAX_SPLITS / 64; ++i) {
        if ((g >> 6) == i) {   // uniform
            T0 = __builtin_amdgcn_readlane(my_wt[i], g & 63);
            T1 = __builtin_amdgcn_readlane(my_wt1[i], g & 63);
        }
    }
    const int r0 = rg * ROWS;
    const int GQ = a.Hq / a.Hkv;

    HW_MARK(0);
    unsigned long long todo = __ballot(lane < a.F && max(T0, my_tb) < min(T1, my_te));

    // One segment = the part of a fragment that lies in this workgroup's tile range.  Opening a segment (decoding the
    // tables, requesting its queries and its first tile) happens before the loop for the first one and at the bottom of
    // the loop for the following ones, so that the requests of the first segment are on their way before the
    // loop-invariant address arithmetic of the tile loop is computed.
    int f = 0, L = 0, lt0 = 0, lt1 = 0;
    bool opens_fragment = false;       // this workgroup owns the fragment's first tile (and writes its rotated queries)
    FragView fv;
    QueryRotation<DT, E, LANEROT ? 1 : ROWS, G::QSTR, PRE> qrot;
    LaneRotation<DT, E, LANEROT ? RB : 1, PRE> lrot;
    int lm = 0;
    [[maybe_unused]] int hw_seg = 0;   // 0 while the first segment is open (selects the timestamp slots of the tuning build)
    TileRegs<DT, E, EV> tr[PF];
    auto open_segment = [&]() {
        f = __builtin_ctzll(todo);
        todo &= todo - 1;
        const int fb = __builtin_amdgcn_readlane(my_tb, f);
        const int fe = __builtin_amdgcn_readlane(my_te, f);
        const int s0 = max(T0, fb), s1 = min(T1, fe);
        L = __builtin_amdgcn_readlane(my_len, f);
        const unsigned long long kp = ((unsigned long long)(unsigned)__builtin_amdgcn_readlane((int)(my_k >> 32), f) << 32) |
                                      (unsigned)__builtin_amdgcn_readlane((int)my_k, f);
        const unsigned long long vp = ((unsigned long long)(unsigned)__builtin_amdgcn_readlane((int)(my_v >> 32), f) << 32) |
                                      (unsigned)__builtin_amdgcn_readlane((int)my_v, f);
        fv = make_view(kp, vp, hkv, L, __builtin_amdgcn_readlane(my_cap, f), G::KROW, G::VROW, reinterpret_cast<unsigned long long>(a.q));
        lt0 = s0 - fb + wv;     // this wave's first tile of the segment (fragment-local)
        lt1 = s1 - fb;
        if constexpr (DEVLEN) lt1 = min(lt1, (L + TILE - 1) / TILE);   // the fragment may be shorter than planned (or empty)
        opens_fragment = s0 == fb;
        // global loads in issue order: query/cos/sin/loc of this fragment first (few), then the first K/V tile; the
        // rotation then waits only for the former while the tile stays in flight
        HW_MARK(hw_seg ? 9 : 6);
        if constexpr (LANEROT) {
            lrot.load(a, f, hkv, r0, GQ, n, q);
        } else {
            qrot.load(a, f, hkv, r0, GQ, tid);
            // (every thread loads, with a clamped row: a load inside a divergent branch would be waited for on the spot)
            lm = a.loc[(size_t)f * a.W * a.S + fast_div(min(r0 + (tid & (ROWS - 1)), a.R - 1), a.magic_gq)];
        }
        HW_MARK(hw_seg ? 10 : 7);
        // the first tile is requested before the prologue, further look-ahead tiles after it: a wave stalls
        // while the memory pipeline accepts its requests, and the prologue should not sit behind that stall
        if (PF > 1) load_tile<DT, E, EV>(tr[0], fv, kslots[0], koff, lt0 * TILE, n, q, lt0 < lt1);
    };
    bool more = todo != 0;
    if (more) open_segment();

    while (more) {
        HW_MARK(hw_seg ? 11 : 1);
        // ---- prologue: rotate the queries of this fragment ----
        u32x4 qreg[QREG ? RB * G::KJ : 1];
        int lim[RB];
        int maxlim = 0, minlim = 0x7fffffff;
        if constexpr (LANEROT) {
            lrot.finish(a, qreg, lim, f, hkv, r0, GQ, L, a.rq != nullptr && opens_fragment && wv == 0, n, q);
        } else {
            // (barriers for LDS only: __syncthreads() would make the K transfers of the tile in flight land first)
            lds_barrier();     // previous segment's readers are done with q_lds / lim_lds
            qrot.finish(a, q_lds, f, hkv, r0, GQ, a.rq != nullptr && opens_fragment, tid);
            // rows that pad the MFMA block get "sees everything": their query is zero and they are never stored,
            // and they must not keep the unmasked fast path from being taken
            if (tid < ROWS) lim_lds[tid] = (r0 + tid < a.R) ? min(L, max(0, lm + 1)) : 0x7fffffff;
            lds_barrier();
            if constexpr (QREG) {
#pragma unroll
                for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                    for (int j = 0; j < G::KJ; ++j)
                        qreg[rb * G::KJ + j] = *reinterpret_cast<const u32x4*>(q_lds + (rb * 16 + n) * G::QSTR + (4 * j + q) * 16);
            }
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) lim[rb] = lim_lds[rb * 16 + n];
        }
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const bool pad = r0 + rb * 16 + n >= a.R;
            maxlim = max(maxlim, pad ? 0 : lim[rb]);
            minlim = min(minlim, lim[rb]);
        }
        maxlim = __builtin_amdgcn_readfirstlane(row_max16(maxlim));
        minlim = __builtin_amdgcn_readfirstlane(row_min16(minlim));
        HW_MARK(hw_seg ? 12 : 2);
#pragma unroll
        for (int i = 1; i < PF - 1; ++i)
            load_tile<DT, E, EV>(tr[i], fv, kslots[i], koff, (lt0 + i * NWAVES) * TILE, n, q, lt0 + i * NWAVES < lt1);

        // ---- stream this wave's tiles: PF buffers, the tile PF-1 steps ahead is requested right before each
        // tile is computed, so its transfer overlaps the arithmetic and the prologue above overlapped the first ----
        // Two loops with one instantiation of the tile arithmetic each: first the groups of PF tiles that every row of
        // the wave sees completely, then the rest.  (With both instantiations in one loop body the compiler merges their
        // accumulators through register copies, 48 v_mov_b64 per tile.)  The fp32 kernels keep the one loop with both: their
        // tiles are MFMA time, and the second loop cost them 0.45 us per launch on the small workloads they serve.
        int lt = lt0;
        constexpr int LAST = (PF - 1) * NWAVES;     // distance of a group's last tile from its first
        if constexpr (G::SZ != 4)
        for (; maxlim > 0 && lt + LAST < lt1 && (lt + LAST + 1) * TILE <= minlim; lt += PF * NWAVES) {
#pragma unroll
            for (int i = 0; i < PF; ++i) {
                const int l = lt + i * NWAVES;
                const int nb = (i + PF - 1) % PF;   // constant after unrolling
                const int ln = l + (PF - 1) * NWAVES;
                load_tile<DT, E, EV>(tr[nb], fv, kslots[nb], koff, ln * TILE, n, q, ln < lt1);
                if constexpr (E > 128) wait_k_landed<G, PF - 1>();
                compute_tile<DT, E, EV, RB, false, QREG, VS>(tr[i], q_lds, qreg, lim, st, l * TILE, n, q, a.sc, kslots[i]);
            }
        }
        for (; lt < lt1; lt += PF * NWAVES) {
#pragma unroll
            for (int i = 0; i < PF; ++i) {
                const int l = lt + i * NWAVES;
                const int t0 = l * TILE;
                const int nb = (i + PF - 1) % PF;
                const int ln = l + (PF - 1) * NWAVES;
                load_tile<DT, E, EV>(tr[nb], fv, kslots[nb], koff, ln * TILE, n, q, ln < lt1);
                if constexpr (E > 128) wait_k_landed<G, PF - 1>();
                const bool live = l < lt1 && t0 < maxlim;
                if (G::SZ == 4 && live && t0 + TILE <= minlim) compute_tile<DT, E, EV, RB, false, QREG, VS>(tr[i], q_lds, qreg, lim, st, t0, n, q, a.sc, kslots[i]);
                else if (live) compute_tile<DT, E, EV, RB, true, QREG, VS>(tr[i], q_lds, qreg, lim, st, t0, n, q, a.sc, kslots[i]);
            }
        }
        more = todo != 0;
        HW_MARK(hw_seg ? 14 : 13);
        hw_seg = 1;
        if (more) open_segment();
    }

    HW_MARK(3);
    // ---- merge the four waves of the workgroup and store the partial of this workgroup ----
    const bool direct = (a.flags & KH_DIRECT) != 0;
    size_t orow[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) orow[rb] = direct ? map_row(a, min(r0 + rb * 16 + n, a.R - 1), hkv, GQ).qrow : 0;
    store_partials<DT, EV, RB, !EXSEP>(st, ex, wv, n, q, tid, a.part_o, a.part_ml, (size_t)(hkv * a.slot_stride + g) * a.R + r0,
                               min(ROWS, a.R - r0), direct, orow);
    HW_MARK(5);

    // rotated queries of zero-length fragments are still part of the operator's visible output
    if (!PRE && a.rq != nullptr && g == 0) {
        unsigned long long empty = __ballot(lane < a.F && my_len == 0);
        while (empty != 0) {
            f = __builtin_ctzll(empty);
            empty &= empty - 1;
            __syncthreads();
            QueryRotation<DT, E, ROWS, G::QSTR, PRE> qempty;
            qempty.load(a, f, hkv, r0, GQ, tid);
            qempty.finish(a, LANEROT ? nullptr : q_lds, f, hkv, r0, GQ, true, tid);
        }
    }
}

// Merge the split-K partials of one (kv head, row): out = sum_g 2^(m_g - M) O_g / sum_g 2^(m_g - M) l_g.
// Latency-bound, so everything a thread needs from global memory (its partial rows and their max/sum pairs) is
// requested in one batch before the first use; each thread then folds its partials with a running reference of
// its own, and the NPG partial groups are combined through LDS.
// RPW = rows per workgroup: with few partials per row (at most 4 * NPG / RPW) a workgroup merges RPW rows side by side,
// each with its share of the partial groups, instead of leaving most of its threads without a partial to load.
template <class DT, int EV, int RPW>
__global__ __launch_bounds__(256) void merge_kernel(const MergeArgs a) {
    typedef typename Elem<DT>::store_t store_t;
    constexpr int V4 = EV / 4;          // threads along the head dim (4 floats each)
    constexpr int NPG = 256 / V4;       // partial groups of the workgroup
    constexpr int GPR = NPG / RPW;      // partial groups per row
    constexpr int UN = 4;               // partials per thread and batch
    static_assert(GPR >= 1 && GPR * RPW == NPG, "the partial groups are dealt evenly to the rows");
    __shared__ __attribute__((aligned(16))) float red[NPG][EV];
    __shared__ float red_m[NPG], red_l[NPG];

    // Workgroups are dealt round-robin over the 8 XCDs.  When the attention kernel kept each kv head on one XCD, merge
    // that head's rows on the same XCD: its partials are then still in that XCD's L2.
    const int nrb = (a.R + RPW - 1) / RPW;                // row blocks per kv head
    int hkv, rblk;
    if (a.xcd_local) {
        const int hpx = a.Hkv >> 3;                       // heads per XCD
        const int x = blockIdx.x & 7, j = blockIdx.x >> 3;
        hkv = x * hpx + j % hpx;
        rblk = j / hpx;
    } else {
        hkv = blockIdx.x / nrb;
        rblk = blockIdx.x - hkv * nrb;
    }
    const int tid = threadIdx.x;
    const int e4 = tid % V4, pg = tid / V4;
    const int rr = pg / GPR, pgl = pg % GPR;               // row within the workgroup, partial group within the row
    const bool live = rblk * RPW + rr < a.R;
    const int r = live ? rblk * RPW + rr : a.R - 1;        // (a row that does not exist re-reads the last one and stores nothing)
    int ns = a.wgs_per_head;
    const float* ml = a.part_ml + ((size_t)hkv * ns * a.R + r) * 2;
    size_t mstride = (size_t)a.R * 2;
    const float* po = a.part_o + ((size_t)hkv * ns * a.R + r) * EV + e4 * 4;
    size_t ostride = (size_t)a.R * EV;
    if (a.row_tab != nullptr) {     // partials by workgroup slot: this row's are in slots first .. first + ns - 1, at row `rl` of each
        // (clamped: the table is device data, and a malformed prefix array of query lengths leaves rows that no entry
        // was written for)
        const int* tab = a.row_tab + ((size_t)hkv * a.R + r) * 2;
        const int x = tab[0];
        const int rl = min(max(tab[1], 0), PLAN_SLOT_ROWS - 1);
        ns = min(max(x >> 16, 0), a.pslots);
        const int first = min(x & 0xffff, a.pslots - ns);
        const size_t base = ((size_t)hkv * a.pslots + first) * PLAN_SLOT_ROWS + rl;
        ml = a.part_ml + base * 2;
        mstride = (size_t)PLAN_SLOT_ROWS * 2;
        po = a.part_o + base * EV + e4 * 4;
        ostride = (size_t)PLAN_SLOT_ROWS * EV;
    }

    float m_run = NEG_BIG, l_run = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = pgl; s0 < ns; s0 += UN * GPR) {
        f32x4 o[UN];
        f32x2 mlv[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int s = s0 + u * GPR;
            const int sc = s < ns ? s : pgl;                // clamp: the loads stay unconditional
            o[u] = *reinterpret_cast<const f32x4*>(po + (size_t)sc * ostride);
            mlv[u] = *reinterpret_cast<const f32x2*>(ml + (size_t)sc * mstride);
            if (s >= ns) mlv[u] = f32x2{NEG_BIG, 0.f};
        }
        float mb = m_run;
#pragma unroll
        for (int u = 0; u < UN; ++u) mb = fmaxf(mb, mlv[u].x);
        const float sc_old = fast_exp2(m_run - mb);
        acc *= sc_old;
        l_run *= sc_old;
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const float w = fast_exp2(mlv[u].x - mb);
            acc += o[u] * w;
            l_run += mlv[u].y * w;
        }
        m_run = mb;
    }
    *reinterpret_cast<f32x4*>(&red[pg][e4 * 4]) = acc;
    if (e4 == 0) {
        red_m[pg] = m_run;
        red_l[pg] = l_run;
    }
    __syncthreads();
    if (pgl == 0 && live) {
        const int g0 = rr * GPR;                           // this row's partial groups: g0 .. g0 + GPR - 1
        float M = red_m[g0];
#pragma unroll
        for (int k = 1; k < GPR; ++k) M = fmaxf(M, red_m[g0 + k]);
        f32x4 tot = {0.f, 0.f, 0.f, 0.f};
        float L = 0.f;
#pragma unroll
        for (int k = 0; k < GPR; ++k) {
            const float w = fast_exp2(red_m[g0 + k] - M);
            tot += *reinterpret_cast<const f32x4*>(&red[g0 + k][e4 * 4]) * w;
            L += red_l[g0 + k] * w;
        }
        const float inv = L > 0.f ? 1.0f / L : 0.f;
        const int GQ = a.Hq / a.Hkv;
        const int ws = r / GQ, gq = r - ws * GQ;
        const int w = ws / a.S, sq = ws - w * a.S;
        const size_t orow = ((size_t)(w * a.Hq + hkv * GQ + gq) * a.S + sq);
        store_t* op = reinterpret_cast<store_t*>(a.out) + orow * EV + e4 * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) op[i] = Elem<DT>::from_float(tot[i] * inv);
        if (a.lse != nullptr && e4 == 0)
            a.lse[orow] = L > 0.f ? (M + __builtin_amdgcn_logf(L)) * 0.69314718055994530942f : -__builtin_inff();
    }
}

// Standalone rotation: out[f,w,h,s,:] = rope(q[w,h,s,:], cos/sin[f,w,s,:])   (src/rope.cuh:2-52)
template <class DT>
__global__ __launch_bounds__(256) void rope_kernel(void* out_, const void* q_, const float* cosv, const float* sinv, int F, int W,
                                                   int Hq, int S, int E, int RotE) {
    typedef typename Elem<DT>::store_t store_t;
    const size_t total = (size_t)F * W * Hq * S * E;
    const store_t* qb = reinterpret_cast<const store_t*>(q_);
    store_t* out = reinterpret_cast<store_t*>(out_);
    const int h = RotE >> 1;
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
        const int e = (int)(idx % E);
        size_t t = idx / E;
        const int s = (int)(t % S);
        t /= S;
        const int hq = (int)(t % Hq);
        t /= Hq;
        const int w = (int)(t % W);
        const int f = (int)(t / W);
        const store_t* qp = qb + (((size_t)w * Hq + hq) * S + s) * E;
        const float x = Elem<DT>::to_float(qp[e]);
        float val = x;
        if (e < RotE) {
            const size_t cs = (((size_t)f * W + w) * S + s) * RotE;
            if (e < h) val = x * cosv[cs + e] - Elem<DT>::to_float(qp[e + h]) * sinv[cs + e];
            else val = x * cosv[cs + e - h] + Elem<DT>::to_float(qp[e - h]) * sinv[cs + e - h];
        }
        out[idx] = Elem<DT>::from_float(val);
    }
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
template <class DT, int E, int EV, bool PRE, bool DEVLEN>
static hipError_t launch_attention_rb(const KernelArgs& ka, int rb, hipStream_t stream) {
    constexpr bool half = Elem<DT>::size == 2;
    if (rb == 1)
        hipLaunchKernelGGL((attention_kernel<DT, E, EV, 1, half ? 2 : 1, half ? 2 : 1, PRE, DEVLEN>), dim3(ka.h.nwg), dim3(NTHREADS), 0,
                           stream, ka);
    else
        hipLaunchKernelGGL((attention_kernel<DT, E, EV, 2, 1, half ? 2 : 1, PRE, DEVLEN>), dim3(ka.h.nwg),
                           dim3(NTHREADS), 0, stream, ka);
    return hipGetLastError();
}

// Head dimension 256: one 16-row block per workgroup and one wave per SIMD.  A K tile is 16 KB per wave, and two row
// blocks of 256-wide accumulators next to the query operands and two V tiles do not fit the register file.
template <class DT, bool PRE, bool DEVLEN>
static hipError_t launch_attention_256(const KernelArgs& ka, int rb, hipStream_t stream) {
    if (rb != 1) return hipErrorInvalidValue;
    hipLaunchKernelGGL((attention_kernel<DT, 256, 256, 1, 1, Elem<DT>::size == 2 ? 2 : 1, PRE, DEVLEN>), dim3(ka.h.nwg), dim3(NTHREADS), 0,
                       stream, ka);
    return hipGetLastError();
}

template <class DT>
static hipError_t launch_attention_dt(const KernelArgs& ka, int E, int rb, int variant, hipStream_t stream) {
    if (E != 64 && E != 128 && E != 256) return hipErrorInvalidValue;
    if (variant == HW_VARIANT_VALU_QK) {     // fused entry, one row block, lengths from the host (checked by the caller)
        constexpr bool half = Elem<DT>::size == 2;
        if (E == 256) return hipErrorInvalidValue;
        if (E == 128)
            hipLaunchKernelGGL((attention_kernel<DT, 128, 128, 1, half ? 2 : 1, half ? 2 : 1, false, false, true>), dim3(ka.h.nwg),
                               dim3(NTHREADS), 0, stream, ka);
        else
            hipLaunchKernelGGL((attention_kernel<DT, 64, 64, 1, half ? 2 : 1, half ? 2 : 1, false, false, true>), dim3(ka.h.nwg),
                               dim3(NTHREADS), 0, stream, ka);
        return hipGetLastError();
    }
    if (ka.h.flags & KH_PREROTATED) {
        if (ka.h.len_dev != nullptr) return hipErrorInvalidValue;   // device-resident lengths exist for the fused entry only
        if (E == 256) return launch_attention_256<DT, true, false>(ka, rb, stream);
        if (E == 128) return launch_attention_rb<DT, 128, 128, true, false>(ka, rb, stream);
        return launch_attention_rb<DT, 64, 64, true, false>(ka, rb, stream);
    }
    if (ka.h.len_dev != nullptr) {
        if (E == 256) return launch_attention_256<DT, false, true>(ka, rb, stream);
        if (E == 128) return launch_attention_rb<DT, 128, 128, false, true>(ka, rb, stream);
        return launch_attention_rb<DT, 64, 64, false, true>(ka, rb, stream);
    }
    if (E == 256) return launch_attention_256<DT, false, false>(ka, rb, stream);
    if (E == 128) return launch_attention_rb<DT, 128, 128, false, false>(ka, rb, stream);
    return launch_attention_rb<DT, 64, 64, false, false>(ka, rb, stream);
}

hipError_t launch_attention(const KernelArgs& ka, int dtype, int E, int rb, int variant, hipStream_t stream) {
    switch (dtype) {
        case 0: return launch_attention_dt<F32>(ka, E, rb, variant, stream);
        case 1: return launch_attention_dt<F16>(ka, E, rb, variant, stream);
        default: return launch_attention_dt<BF16>(ka, E, rb, variant, stream);
    }
}

template <class DT, int EV>
static hipError_t launch_merge_ev(const MergeArgs& ma, hipStream_t stream) {
    constexpr int NPG = 256 / (EV / 4);
    // rows per workgroup: as many as leave every row one batch of four partials per thread group
    const int ns = ma.wgs_per_head;
    auto go = [&](auto rpw_tag) {
        constexpr int RPW = decltype(rpw_tag)::value;
        const int blocks = ma.Hkv * ((ma.R + RPW - 1) / RPW);
        hipLaunchKernelGGL((merge_kernel<DT, EV, RPW>), dim3(blocks), dim3(256), 0, stream, ma);
    };
    if constexpr (NPG >= 8) {       // (eight rows side by side need eight thread groups: not at head dimension 256)
        if (ns <= 4) {
            go(std::integral_constant<int, 8>{});
            return hipGetLastError();
        }
    }
    if (ns <= 4 * (NPG / 4)) go(std::integral_constant<int, 4>{});
    else if (ns <= 4 * (NPG / 2)) go(std::integral_constant<int, 2>{});
    else go(std::integral_constant<int, 1>{});
    return hipGetLastError();
}

template <class DT>
static hipError_t launch_merge_dt(const MergeArgs& ma, int EV, hipStream_t stream) {
    if (EV == 256) return launch_merge_ev<DT, 256>(ma, stream);
    if (EV == 128) return launch_merge_ev<DT, 128>(ma, stream);
    return launch_merge_ev<DT, 64>(ma, stream);
}

hipError_t launch_merge(const MergeArgs& ma, int dtype, int EV, hipStream_t stream) {
    switch (dtype) {
        case 0: return launch_merge_dt<F32>(ma, EV, stream);
        case 1: return launch_merge_dt<F16>(ma, EV, stream);
        default: return launch_merge_dt<BF16>(ma, EV, stream);
    }
}

hipError_t launch_rope(void* out, const void* q, const float* cosv, const float* sinv, int dtype, int F, int W, int Hq, int S,
                       int E, int RotE, hipStream_t stream) {
    const size_t total = (size_t)F * W * Hq * S * E;
    int blocks = (int)((total + 255) / 256);
    if (blocks > 4096) blocks = 4096;
    if (blocks < 1) blocks = 1;
    switch (dtype) {
        case 0: hipLaunchKernelGGL((rope_kernel<F32>), dim3(blocks), dim3(256), 0, stream, out, q, cosv, sinv, F, W, Hq, S, E, RotE); break;
        case 1: hipLaunchKernelGGL((rope_kernel<F16>), dim3(blocks), dim3(256), 0, stream, out, q, cosv, sinv, F, W, Hq, S, E, RotE); break;
        default: hipLaunchKernelGGL((rope_kernel<BF16>), dim3(blocks), dim3(256), 0, stream, out, q, cosv, sinv, F, W, Hq, S, E, RotE); break;
    }
    return hipGetLastError();
}

}  // namespace hw

#ifdef HW_CLOCKS
extern "C" int hw_debug_read_clocks(unsigned long long* host, size_t n) {
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(hw::hw_clock_buf), n * sizeof(unsigned long long));
}
#endif
