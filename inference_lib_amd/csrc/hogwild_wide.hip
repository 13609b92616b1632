// Hogwild! fragmented-KV attention for many query rows per kv head (several tokens per worker, many workers, wide GQA
// groups): the shape where a decode step turns into a small prefill.  gfx950 (MI355X, CDNA4, wave64), 16-bit types.
//
// One workgroup = one kv head x one contiguous range of 32-token tiles x up to 128 query rows, eight waves: four groups
// of 32 rows (two 16-row MFMA blocks), and the two waves of a group -- the two waves of one SIMD -- take every other
// tile.  A tile is brought into LDS once per workgroup -- K and V by direct global->LDS transfers, every wave issuing its
// share -- and read from there by the four waves whose turn it is.  What bounds the narrow kernel on such shapes is the
// rate at which one CU can take data in (about 16 B/clk through the vector memory path, whatever cache answers): with
// 32-row workgroups every group of 32 rows streams the whole KV through its CU again, four times for 128 rows.  Here a
// CU takes every byte in once and spreads it through LDS (a wave reads 16 KB per tile it multiplies out of 128 B/clk of
// LDS bandwidth; with one wave per SIMD taking every tile the arithmetic of a tile had nothing to run beside, with two
// waves per SIMD that both take every tile the LDS reads double).
//
// The tiles rotate through a ring of NS LDS slots in steps of PAR = 2 tiles, one for each wave of a group.  One barrier
// per step: a wave waits for its own transfers of the step, all waves meet, the step is complete in LDS; and since every
// wave has then left the step before behind, its slots are free for the request issued right behind the barrier (NS / PAR
// - 1 steps are in flight or being multiplied).  The transfers are issued from inline assembly and waited for by hand
// (see lds_transfer).
// The two waves of a group add up their partial sums through LDS at the end (each takes one 16-row block of the 32
// rows); rows of different groups are different rows.  Every wave then stores the partial (unnormalised output, running
// max, sum) of its block, and the merge kernel of the narrow path (merge_kernel) finishes the job.
//
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/hogwild_hip.h"
#include "hogwild_kernels.h"

namespace hw {

// Phase timestamps of the 128-row kernels for tuning (the first four waves of a workgroup); compiled in only with
// -DHW_CLOCKS (never in the shipped library).
#ifdef HW_CLOCKS
__device__ unsigned long long hw_wide_clock_buf[1024 * 4 * 16];
#define HW_MARK(i)                                                                                  \
    do {                                                                                            \
        if ((threadIdx.x & 63) == 0 && threadIdx.x < 256 && blockIdx.x < 1024)                                        \
            hw_wide_clock_buf[(blockIdx.x * 4 + (threadIdx.x >> 6)) * 16 + (i)] = wall_clock64();    \
    } while (0)
#define HW_NOTE(i, v)                                                                               \
    do {                                                                                            \
        if ((threadIdx.x & 63) == 0 && threadIdx.x < 256 && blockIdx.x < 1024)                                        \
            hw_wide_clock_buf[(blockIdx.x * 4 + (threadIdx.x >> 6)) * 16 + (i)] = (unsigned long long)(v); \
    } while (0)
#else
#define HW_MARK(i) do { } while (0)
#define HW_NOTE(i, v) do { } while (0)
#endif

}  // namespace hw

#include "hogwild_device.h"

namespace hw {


constexpr int WIDE_ROWS = 128;      // query rows per workgroup: 32 per wave

// A slice of device memory as a raw buffer descriptor (base, stride 0, size in bytes, flags): reads beyond the size
// return zero.  Held as plain words: the transfers below are issued from inline assembly.
__device__ __forceinline__ u32x4 raw_descriptor(unsigned long long base, unsigned bytes) {
    u32x4 d;
    d.x = __builtin_amdgcn_readfirstlane((u32)base);
    d.y = __builtin_amdgcn_readfirstlane((u32)(base >> 32) & 0xffffu);
    d.z = __builtin_amdgcn_readfirstlane(bytes);
    d.w = 0x00020000u;
    return d;
}
// One 1 KB global->LDS transfer (lane l: 16 bytes from descriptor offset `voffset` to LDS byte `lds` + 16 l), non-temporal.
// Issued from inline assembly on purpose: the compiler waits for every transfer it knows of before a read of LDS it
// cannot prove disjoint, which would empty the look-ahead queue at every tile; these it does not know of, and the kernel
// waits for them itself (s_waitcnt vmcnt before the barrier of each tile).  Loads complete in order, so a compiler-
// generated wait for one of its own loads can only become longer through them, never too short.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"   // m0 is a reserved register: it is set and used inside the one statement
__device__ __forceinline__ void lds_transfer(const u32x4& desc, unsigned lds, unsigned voffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen nt lds" ::"s"(lds), "v"(voffset), "s"(desc) : "m0", "memory");
}
#pragma clang diagnostic pop

// One wave's share of a tile's transfers: TPW 1 KB pieces of ONE image (the first half of the waves fill K, the second
// half V), into LDS bytes `slot` + 1024 j.  `tile` = byte offset of the tile in the kv head's slice (OOB_OFFSET for a
// tile that does not exist: the same number of transfers, no memory traffic, zeros in LDS).
template <int TPW>
__device__ __forceinline__ void wide_request(const u32x4& desc, unsigned slot, unsigned tile, const unsigned* off) {
#pragma unroll
    for (int j = 0; j < TPW; ++j) lds_transfer(desc, slot + j * 1024, tile + off[j]);
}

__device__ __forceinline__ unsigned lds_address(const void* p) {
    return __builtin_amdgcn_readfirstlane((unsigned)(size_t)HW_LDS_PTR(p));
}

// Query rotation of one fragment for the 128 rows of a workgroup (the role of QueryRotation in the narrow kernel).  The
// rows of one (worker, token) pair share their cos/sin table row, and with 128 rows per workgroup loading it per query
// row made the prologue the most expensive part of the kernel (a CU takes in ~16 B/clk: 64 KB of table rows against
// 32 KB of queries).  Here the distinct table rows of the workgroup go through LDS once (first halves only: both halves
// of the rotation read cos/sin at the first-half index, src/rope.cuh:30-46), CSMAX of them; a workgroup whose rows span
// more (worker, token) pairs than that (GQA ratio below 4) cannot use it and takes the per-row path.
template <class DT, int E, int QSTR, int NT>
struct WideRotation {
    static constexpr int SZ = Elem<DT>::size;
    static constexpr int CH = Chunk<DT>::CH;
    static constexpr int IPR = E / (2 * CH);                                  // chunk pairs per row
    static constexpr int NIT = (WIDE_ROWS * IPR + NT - 1) / NT;   // chunk pairs per thread
    static constexpr int CSMAX = 36;                                          // table rows staged per workgroup
    static constexpr int CPW = E / 2 / 4;                                     // float4 per half table row
    static constexpr int NCS = (CSMAX * 2 * CPW + NT - 1) / NT;   // table float4 per thread
    static constexpr int CS_FLOATS = CSMAX * E;                               // [row][cos half | sin half]

    u32x4 xa[NIT], xb[NIT];
    f32x4 tab[NCS];

    // global loads: the queries of this thread's chunk pairs (the same for every fragment) ...
    __device__ __forceinline__ void load_queries(const DevHeader& a, int hkv, int r0, int GQ, int tid) {
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int item = tid + it * NT;
            const int rr = item / IPR, slot = item % IPR;
            const int r = (item < WIDE_ROWS * IPR && r0 + rr < a.R) ? r0 + rr : r0;
            const RowMap rm = map_row(a, r, hkv, GQ);
            const HW_GLOBAL char* qp = a.q + rm.qrow * E * SZ;
            xa[it] = *reinterpret_cast<const HW_GLOBAL u32x4*>(qp + slot * 16);
            xb[it] = *reinterpret_cast<const HW_GLOBAL u32x4*>(qp + (slot + IPR) * 16);
        }
    }
    // ... and its share of fragment f's table rows ws_lo .. ws_lo + nws - 1
    __device__ __forceinline__ void load_tables(const DevHeader& a, int f, int tid, int ws_lo, int nws) {
#pragma unroll
        for (int k = 0; k < NCS; ++k) {
            const int item = tid + k * NT;
            const int wi = min(item / (2 * CPW), nws - 1), part = item % (2 * CPW);      // beyond the last row: re-read it
            const HW_GLOBAL float* src = (part < CPW ? a.cos : a.sin) + ((size_t)f * a.W * a.S + ws_lo + wi) * E + (part % CPW) * 4;
            tab[k] = *reinterpret_cast<const HW_GLOBAL f32x4*>(src);
        }
    }

    // table rows into LDS (a barrier must follow before rotate())
    __device__ __forceinline__ void stage(float* cs_lds, int tid, int nws) const {
#pragma unroll
        for (int k = 0; k < NCS; ++k) {
            const int item = tid + k * NT;
            if (item < nws * 2 * CPW) *reinterpret_cast<f32x4*>(cs_lds + item * 4) = tab[k];
        }
    }

    __device__ __forceinline__ void rotate(const DevHeader& a, char* q_lds, const float* cs_lds, int f, int hkv, int r0, int GQ, bool write_rq,
                                           int tid, int ws_lo) const {
        const size_t fstride = (size_t)a.W * a.Hq * a.S * E;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int item = tid + it * NT;
            const int rr = item / IPR, slot = item % IPR;
            if (item >= WIDE_ROWS * IPR) continue;
            char* lrow = q_lds + rr * QSTR;
            const bool pad = r0 + rr >= a.R;
            const RowMap rm = map_row(a, pad ? r0 : r0 + rr, hkv, GQ);
            const float* cs = cs_lds + (rm.ws - ws_lo) * E + slot * CH;
            float x1[CH], x2[CH], y1[CH], y2[CH];
            Chunk<DT>::unpack(xa[it], x1);
            Chunk<DT>::unpack(xb[it], x2);
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                const float c = cs[i], sv = cs[E / 2 + i];
                y1[i] = x1[i] * c - x2[i] * sv;
                y2[i] = x2[i] * c + x1[i] * sv;
            }
            const u32x4 z = {0, 0, 0, 0};
            const u32x4 ya = Chunk<DT>::pack(y1), yb = Chunk<DT>::pack(y2);
            *reinterpret_cast<u32x4*>(lrow + slot * 16) = pad ? z : ya;
            *reinterpret_cast<u32x4*>(lrow + (slot + IPR) * 16) = pad ? z : yb;
            if (write_rq && !pad) {
                HW_GLOBAL char* rqp = a.rq + (f * fstride + rm.qrow * E) * SZ;
                *reinterpret_cast<HW_GLOBAL u32x4*>(rqp + slot * 16) = ya;
                *reinterpret_cast<HW_GLOBAL u32x4*>(rqp + (slot + IPR) * 16) = yb;
            }
        }
    }
};

template <class DT, int E, int EV, int NS, bool PRE, int NW, int PAR>
__global__ __launch_bounds__(NW * 64, 1) void attention_wide_kernel(const KernelArgs args) {
    typedef Geo<DT, E, EV> G;
    constexpr int NT = NW * 64;                 // threads per workgroup
    constexpr int NRW = NW / PAR;               // waves that differ in their rows; PAR waves share the rows and alternate on the tiles
    constexpr int RB = WIDE_ROWS / 16 / NRW;    // 16-row blocks per wave
    constexpr int WROWS = RB * 16;              // rows per wave
    constexpr int TPR = NT / WIDE_ROWS;         // threads per row where a row is handled by a group of threads
    constexpr int NSTEP = NS / PAR;             // ring slots in steps of PAR tiles (one barrier per step)
    constexpr int DP = NSTEP - 1;               // steps requested ahead
    constexpr int KBYTES = G::KSTAGE;           // K image of a tile in LDS
    constexpr int VBYTES = TILE * G::VROW;      // V image
    constexpr int TPW = (KBYTES + VBYTES) / 1024 / NW;   // 1 KB transfers each wave issues per tile
    constexpr int TPS = PAR * TPW;              // ... per step
    constexpr int SLOT = KBYTES + VBYTES;
    static_assert(G::SZ == 2 && KBYTES == VBYTES && TPW >= 1 && (KBYTES / 1024) % TPW == 0 && NS % PAR == 0 && DP >= 1 && RB >= 1 &&
                      NW % PAR == 0 && (PAR == 1 || PAR == 2),
                  "16-bit types; a wave's transfers belong to one image");

    __shared__ __attribute__((aligned(16))) char q_lds[WIDE_ROWS * G::QSTR];
    __shared__ int lim_lds[WIDE_ROWS];
    typedef WideRotation<DT, E, G::QSTR, NT> WRot;
    __shared__ __attribute__((aligned(16))) float cs_lds[PRE ? 4 : WRot::CS_FLOATS];
    // ring slots: [K image | V image]; K is swizzled like in the narrow kernel, V is a plain row-major image
    __shared__ __attribute__((aligned(16))) char ring[NS * SLOT];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rw = wv % NRW;                    // which rows
    const int par = wv / NRW;                   // which tile of a step
    const int n = lane & 15;
    const int q = lane >> 4;
    HW_MARK(8);

    // the kernel arguments in one burst (see attention_kernel)
    const int fl = lane & (MAXF - 1);
    const unsigned long long my_k = reinterpret_cast<unsigned long long>(args.frag.k[fl]);
    const unsigned long long my_v = reinterpret_cast<unsigned long long>(args.frag.v[fl]);
    const FragTable::LenCap my_lc = args.frag.lc[fl];
    const int my_len = my_lc.len;
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
    // this wave's share of a tile's transfers.  A transfer writes LDS linearly (lane l -> base + 16 l); the K swizzle is
    // applied on the global side (see k_lane_offsets)
    const bool k_wave = wv < NW / 2;
    const int first = (k_wave ? wv : wv - NW / 2) * TPW;          // first 1 KB piece of the image
    unsigned off[TPW];
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
        const int p = (first + j) * 64 + lane;
        const int row = p / G::CPR, slot = p % G::CPR;
        const int key = G::CPR >= 16 ? (row & 15) : ((row >> 1) & (G::CPR - 1));
        off[j] = k_wave ? row * G::KROW + ((slot ^ key) << 4) : row * G::VROW + ((slot ^ (2 * vimg_segment_key<G::VROW>(row))) << 4);
    }
    const unsigned long long my_image_ptr = k_wave ? my_k : my_v;   // lane f: this wave's image of fragment f
    const int image_row = k_wave ? G::KROW : G::VROW;               // bytes per token in it
    const unsigned my_image = lds_address(ring) + (k_wave ? 0 : KBYTES) + first * 1024;   // in slot 0
    WaveState<RB, G::NOC> st;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        st.m[rb] = NEG_BIG;
        st.l[rb] = 0.f;
#pragma unroll
        for (int c = 0; c < G::NOC; ++c) st.o[rb][c] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    st.fresh = true;
    unsigned voff[G::NOC];                             // this lane's positions in a V image (transposed reads)
    vtr_lane_offsets<G::VROW>(voff, lane);
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(hb.lo), "+s"(hb.hi) : : "memory");
    const DevHeader a = __builtin_bit_cast(DevHeader, hb);
    HW_MARK(0);

    int bid = blockIdx.x;
    if (a.flags & KH_XCD_REMAP) bid = (bid & 7) * (a.nwg >> 3) + (bid >> 3);
    const int hg = fast_div(bid, a.magic_nrg);
    const int rg = bid - hg * a.nrg;
    const int hkv = fast_div(hg, a.magic_wg);
    const int g = hg - hkv * a.wgs_per_head;
    int T0 = 0, T1 = 0;
#pragma unroll
    for (int i = 0; i < MAX_SPLITS / 64; ++i) {
        if ((g >> 6) == i) {
            T0 = __builtin_amdgcn_readlane(my_wt[i], g & 63);
            T1 = __builtin_amdgcn_readlane(my_wt1[i], g & 63);
        }
    }
    const int r0 = rg * WIDE_ROWS;              // first row of the workgroup
    const int w0 = r0 + rw * WROWS;             // first row of this wave
    const int GQ = a.Hq / a.Hkv;
    // (worker, token) pairs the rows of this workgroup belong to
    const int ws_lo = fast_div(r0, a.magic_gq);
    const int nws = fast_div(min(r0 + WIDE_ROWS, a.R) - 1, a.magic_gq) - ws_lo + 1;
    const bool staged = !PRE && nws <= WRot::CSMAX;          // uniform over the workgroup
    // The queries to rotate are the same for every fragment: they are requested here, before the workgroup's tile range
    // and first fragment are worked out, and are on their way while that happens.
    WRot wrot;
    const bool early_queries = staged;
    if (early_queries) wrot.load_queries(a, hkv, r0, GQ, tid);

    HW_MARK(10);
    unsigned long long todo = __ballot(lane < a.F && max(T0, my_tb) < min(T1, my_te));
    int f = 0, L = 0, lt0 = 0, lt1 = 0;
    bool opens_fragment = false;
    u32x4 view = {0, 0, 0, 0};                               // this wave's image of the current fragment (K or V slice)
    [[maybe_unused]] QueryRotation<DT, E, WIDE_ROWS, G::QSTR, true, NT> qrot;     // pre-rotated queries: a copy into LDS
    int lm = 0;

    // this wave's share of the PAR tiles of the step that starts at tile `lt` (fragment-local) into step slot `ss`; a tile
    // that does not exist is requested out of range: the same number of transfers, no memory traffic, zeros in LDS
    auto request = [&](int ss, int lt) {
#pragma unroll
        for (int pp = 0; pp < PAR; ++pp) {
            const unsigned tile_bytes = (unsigned)((lt + pp) * TILE * image_row);
            wide_request<TPW>(view, __builtin_amdgcn_readfirstlane(my_image + (ss * PAR + pp) * SLOT), lt + pp < lt1 ? tile_bytes : OOB_OFFSET, off);
        }
    };

    auto open_segment = [&](bool queries_requested) {
        f = __builtin_ctzll(todo);
        todo &= todo - 1;
        const int fb = __builtin_amdgcn_readlane(my_tb, f);
        const int fe = __builtin_amdgcn_readlane(my_te, f);
        const int s0 = max(T0, fb), s1 = min(T1, fe);
        L = __builtin_amdgcn_readlane(my_len, f);
        const unsigned long long base = ((unsigned long long)(unsigned)__builtin_amdgcn_readlane((int)(my_image_ptr >> 32), f) << 32) |
                                        (unsigned)__builtin_amdgcn_readlane((int)my_image_ptr, f);
        const int cap = __builtin_amdgcn_readlane(my_cap, f);
        view = raw_descriptor(base + (unsigned long long)hkv * cap * image_row, (unsigned)(L * image_row));
        lt0 = s0 - fb;
        lt1 = s1 - fb;
        opens_fragment = s0 == fb;
        // The first step is requested before the queries: the compiler's wait for the query loads then also waits for it
        // (loads complete in order), which costs nothing, its tiles being needed first anyway.  The other look-ahead
        // steps follow when the queries have arrived, so that the rotation does not wait for them as well.
        request(0, lt0);
        HW_MARK(11);
        // (the thread index as the compiler cannot see through it: what is derived from it -- rows, addresses of the
        // queries -- is then formed per segment instead of once in front of the loop over the segments, from where it
        // would stay in registers across the tile loops, which have none to spare)
        int tids = tid;
        asm volatile("" : "+v"(tids));
        if constexpr (PRE) {
            qrot.load(a, f, hkv, r0, GQ, tids);
        } else if (staged) {
            if (!queries_requested) wrot.load_queries(a, hkv, r0, GQ, tids);
            wrot.load_tables(a, f, tids, ws_lo, nws);
        }
        // the bound of row tid / TPR (TPR threads per row, all load: keeps the load unconditional)
        lm = a.loc[(size_t)f * a.W * a.S + fast_div(min(r0 + tids / TPR, a.R - 1), a.magic_gq)];
    };
    bool more = todo != 0;
    if (more) open_segment(early_queries);
    HW_MARK(6);
    bool hw_first = true;

    while (more) {
        __syncthreads();   // previous segment's readers are done with q_lds / lim_lds
        if (hw_first) HW_MARK(7);
        int tids = tid;        // (see open_segment)
        asm volatile("" : "+v"(tids));
        // Every load of open_segment is waited for here, in a form the compiler sees: it waits for a load where its result
        // is first used and counts only the loads it knows of, so a wait that it places further down -- for the bound
        // below, the last load of open_segment -- would also wait for the look-ahead steps requested in between.
        // (Nothing is lost: the queries are needed now, and the first step was requested before them.)
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        int limv = (r0 + tids / TPR < a.R) ? min(L, max(0, lm + 1)) : 0x7fffffff;   // by every thread, see paged_wide_kernel
        asm volatile("" : "+v"(limv));
        if (!PRE && staged) {
            wrot.stage(cs_lds, tids, nws);
            if (hw_first) HW_MARK(13);
            // The barrier above has waited for every load of open_segment: the other look-ahead steps can be requested
            // here, ahead of the rotation arithmetic, which waits for nothing from memory any more.  (An LDS-only barrier
            // again: __syncthreads() would wait for the requests just issued.)
#pragma unroll
            for (int i = 1; i < DP; ++i) request(i, lt0 + i * PAR);
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            if (hw_first) HW_MARK(14);
            wrot.rotate(a, q_lds, cs_lds, f, hkv, r0, GQ, a.rq != nullptr && opens_fragment, tids, ws_lo);
        } else if constexpr (PRE) {
            qrot.finish(a, q_lds, f, hkv, r0, GQ, false, tids);
        } else {
            // too many (worker, token) pairs for the staged tables (GQA ratio below 4): every row loads its own table row,
            // here and not ahead of time in open_segment, so that the registers of this path are not held across the tile
            // loops of the common one
            QueryRotation<DT, E, WIDE_ROWS, G::QSTR, false, NT> qslow;
            qslow.load(a, f, hkv, r0, GQ, tids);
            qslow.finish(a, q_lds, f, hkv, r0, GQ, a.rq != nullptr && opens_fragment, tids);
            // (said once more where the compiler sees it: without it, it takes this path's loads for outstanding on the
            // other path of the next segment and waits there, in the middle of the rotation, for "everything")
            __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        }
        if (tids % TPR == 0) lim_lds[tids / TPR] = limv;
        if (hw_first) HW_MARK(12);
        // q_lds and lim_lds become visible: a barrier for LDS only.  __syncthreads() would also wait for the stores of
        // the rotated queries to be acknowledged by memory, which nobody here depends on.
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (hw_first) HW_MARK(1);

        // this wave's query operands and mask bounds
        u32x4 qreg[RB * G::KJ];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int j = 0; j < G::KJ; ++j)
                qreg[rb * G::KJ + j] = *reinterpret_cast<const u32x4*>(q_lds + (rw * WROWS + rb * 16 + n) * G::QSTR + (4 * j + q) * 16);
        int lim[RB];
        int maxlim = 0, minlim = 0x7fffffff;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            lim[rb] = lim_lds[rw * WROWS + rb * 16 + n];
            const bool pad = w0 + rb * 16 + n >= a.R;
            maxlim = max(maxlim, pad ? 0 : lim[rb]);
            minlim = min(minlim, lim[rb]);
        }
        maxlim = __builtin_amdgcn_readfirstlane(row_max16(maxlim));
        minlim = __builtin_amdgcn_readfirstlane(row_min16(minlim));
        if (PRE || !staged) {
#pragma unroll
            for (int i = 1; i < DP; ++i) request(i, lt0 + i * PAR);
        }

        {
            // A step = PAR tiles behind one barrier, one for each of the waves that share their rows.  Two loops, one
            // instantiation of the tile arithmetic in each: first the steps in which every row of this wave sees its tile
            // completely, then the rest.  With both instantiations in one loop body the compiler merges their accumulators
            // through copies (48 v_mov_b64 per tile).  The waves of a workgroup may change loops at different steps; each
            // still passes one barrier per step.
            int ss = 0;                                   // step slot of the current step
            int l = lt0;                                  // its first tile
            auto arrive = [&]() {
                // this wave's transfers of the step have landed (the DP - 1 steps requested since may stay in flight: loads
                // complete in order), then every wave's.  Behind the barrier the slots of the step before are free:
                // request step + DP into them.
                asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((DP - 1) * TPS) : "memory");
                request(ss == 0 ? NSTEP - 1 : ss - 1, l + DP * PAR);
                if (hw_first) { HW_MARK(2); hw_first = false; }
            };
            const int lfast = maxlim > 0 ? min(lt1, minlim / TILE) : lt0;
#pragma unroll 1
            for (; l + par < lfast; l += PAR) {
                arrive();
                const char* slot = ring + (ss * PAR + par) * SLOT;
                compute_tile<DT, E, EV, RB, false, true, false, true>(TileRegs<DT, E, EV>(), q_lds, qreg, lim, st, (l + par) * TILE, n, q, a.sc, slot, slot + KBYTES, voff);
                ss = ss + 1 == NSTEP ? 0 : ss + 1;
            }
#pragma unroll 1
            for (; l < lt1; l += PAR) {
                arrive();
                if (l + par < lt1 && (l + par) * TILE < maxlim) {
                    const char* slot = ring + (ss * PAR + par) * SLOT;
                    compute_tile<DT, E, EV, RB, true, true, false, true>(TileRegs<DT, E, EV>(), q_lds, qreg, lim, st, (l + par) * TILE, n, q, a.sc, slot, slot + KBYTES, voff);
                }
                ss = ss + 1 == NSTEP ? 0 : ss + 1;
            }
        }
        // the requests behind the last tile (they fetched nothing) must have landed before the ring is used again
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        more = todo != 0;
        if (more) {
            __syncthreads();   // every wave is done with the ring
            open_segment(false);
        }
    }

    // ---- The PAR waves that share their rows hold a partial sum each: block rb of the rows goes to wave rb % PAR of them
    // through LDS, lane for lane in the accumulator layout, and is added up there.  Then every wave stores the blocks it
    // owns.  The accumulator layout scatters a row over the lanes in 16-byte pieces; written like that, a partial (17 MB
    // per launch at 128 rows x 32 workgroups x 8 heads) would reach memory as a million partial-line writes.  So each
    // 16-row block goes through LDS once more -- all of this in the ring, which no tile needs any more -- and leaves as
    // whole rows, 1 KB per store. ----
    {
        constexpr int OSTR = EV + 4;                                  // floats per staged row (padded against bank conflicts)
        constexpr int REGION = 16 * OSTR;                             // floats per wave: a staged 16-row block, or a block in accumulator layout
        static_assert(G::NOC * 64 * 4 <= REGION && (NW * REGION + NW * 64 * 2) * 4 <= NS * SLOT, "the blocks of all waves fit into the ring");
        HW_MARK(3);
        __syncthreads();                                              // every wave has left the last tile
        HW_MARK(4);
        float* const regions = reinterpret_cast<float*>(ring);
        float* const mls = regions + NW * REGION;
        if constexpr (PAR > 1) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                const int owner = rw + (rb % PAR) * NRW;
                if (owner != wv) {
#pragma unroll
                    for (int c = 0; c < G::NOC; ++c) *reinterpret_cast<f32x4*>(regions + owner * REGION + (c * 64 + lane) * 4) = st.o[rb][c];
                    *reinterpret_cast<f32x2*>(mls + (owner * 64 + lane) * 2) = f32x2{st.m[rb], st.l[rb]};
                }
            }
            __syncthreads();
        }
        float* stage = regions + wv * REGION;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            if (rw + (rb % PAR) * NRW != wv) continue;                // uniform over the wave
            if constexpr (PAR > 1) {
                const f32x2 oml = *reinterpret_cast<const f32x2*>(mls + (wv * 64 + lane) * 2);
                const float mnew = fmaxf(st.m[rb], oml.x);
                const float mine = exp2f(st.m[rb] - mnew), theirs = exp2f(oml.x - mnew);
#pragma unroll
                for (int c = 0; c < G::NOC; ++c) {
                    const f32x4 o2 = *reinterpret_cast<const f32x4*>(stage + (c * 64 + lane) * 4);
#pragma unroll
                    for (int i = 0; i < 4; ++i) st.o[rb][c][i] = st.o[rb][c][i] * mine + o2[i] * theirs;
                }
                st.l[rb] = st.l[rb] * mine + oml.y * theirs;
                st.m[rb] = mnew;
            }
            const float lsum = quarter_sum(st.l[rb]);
            const int row0 = w0 + rb * 16;                            // first row of the block
            const size_t prow0 = (size_t)(hkv * a.slot_stride + g) * a.R + row0;
#pragma unroll
            for (int c = 0; c < G::NOC; ++c)              // block c, accumulator rows 4q .. 4q+3 = elements 16c + 4q ..
                *reinterpret_cast<f32x4*>(stage + n * OSTR + 16 * c + 4 * q) = st.o[rb][c];
            if (q == 0 && row0 + n < a.R) *reinterpret_cast<HW_GLOBAL f32x2*>(a.part_ml + (prow0 + n) * 2) = f32x2{st.m[rb], lsum};
            // (one wave: the LDS writes above are complete before the reads below are issued, in program order, and
            // the reads before the next block's writes)
            const int nvalid = min(16, a.R - row0);                   // rows of the block that exist
            HW_GLOBAL float* dst = a.part_o + prow0 * EV;
#pragma unroll
            for (int ps = 0; ps < 16 * EV / 256; ++ps) {              // 64 lanes x 4 floats per pass
                const int idx = ps * 256 + lane * 4;
                const int rr = idx / EV, e = idx % EV;
                if (rr < nvalid) *reinterpret_cast<HW_GLOBAL f32x4*>(dst + idx) = *reinterpret_cast<const f32x4*>(stage + rr * OSTR + e);
            }
        }
    }

    HW_MARK(5);

    // rotated queries of zero-length fragments are still part of the operator's visible output
    if (!PRE && a.rq != nullptr && g == 0) {
        unsigned long long empty = __ballot(lane < a.F && my_len == 0);
        while (empty != 0) {
            f = __builtin_ctzll(empty);
            empty &= empty - 1;
            __syncthreads();
            QueryRotation<DT, E, WIDE_ROWS, G::QSTR, PRE, NT> qempty;
            qempty.load(a, f, hkv, r0, GQ, tid);
            qempty.finish(a, q_lds, f, hkv, r0, GQ, true, tid);
        }
    }
}

// One 1 KB global->LDS transfer with a 64-bit address per lane (the paged cache has no contiguous slice a buffer
// descriptor could bound): lane l brings 16 bytes from `src` to LDS byte `lds` + 16 l, non-temporal.  Issued from inline
// assembly and waited for by hand, like lds_transfer.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void lds_transfer_flat(unsigned lds, unsigned long long src) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(lds), "v"(src) : "m0", "memory");
}
#pragma clang diagnostic pop

// The split of a packed-query launch, decided on the device (query lengths and KV lengths are device tensors,
// src/binding.cu:144-181) -- by every workgroup for itself, in its prologue: the inputs are a few hundred bytes that
// all workgroups read, and a planning kernel in front of the launch cost 5.8 us plus the gap between two launches.
// One thread per sequence and then per row group (at most PLAN_MAX_GROUPS of either; the host sends larger batches
// down the unplanned path).  Every kv head has `pslots` workgroup slots.  A row group = up to 128 rows of one sequence;
// its work is its sequence's tiles times the cost of a tile (a group of at most 64 rows keeps one wave per SIMD busy
// instead of two: 0.67 against 0.88 us per tile measured, 3 : 4).  Every group takes one slot and a share of the others in
// proportion to its work (what the rounding leaves over goes to the groups with the most work per slot), four tiles per
// slot at least; slots are numbered through the groups in order.  Returns what slot `item` does
// (found = false: nothing), and -- for the workgroup that holds a group's first slot -- tells the merge kernel through
// the kv head's row table where the partial sums of the group's rows lie (a table per kv head, although they are all the
// same: the merge of a head runs on the XCD whose workgroups wrote the head's partial sums and table, and finds both in
// that XCD's L2).
struct PlanSlot {
    int w, rg, qs, qe, split, ns;
    bool found;
};
// Where the merge finds the partial sums of a row: {first slot | slots << 16, row within the slot}, written by the
// workgroup that holds a row group's first slot; rows behind the last sequence (its query range ends at last_qe) have
// none: the workgroup of slot 0 writes zeros for them, and the merge gives them zeros.
template <int NTW>
__device__ __forceinline__ void plan_row_table(const PagedDevHeader& ph, const PlanSlot& r, int item, int hkv, int GQ, int tid, int last_qe) {
    HW_GLOBAL int* row_tab = reinterpret_cast<HW_GLOBAL int*>(ph.part_ml + (size_t)ph.Hkv * ph.nitems * PLAN_SLOT_ROWS * 2) + (size_t)hkv * ph.R * 2;
    if (r.found && r.split == 0) {
        const int nrows = min((r.qe - r.qs) * GQ - r.rg * WIDE_ROWS, WIDE_ROWS);
        const int row = r.qs * GQ + r.rg * WIDE_ROWS + tid;
        if (tid < nrows && row < ph.R) {
            row_tab[2 * row] = (item - r.split) | (r.ns << 16);
            row_tab[2 * row + 1] = tid;
        }
    }
    if (item == 0) {
        const int covered = min(last_qe * GQ, ph.R);
        for (int i = covered * 2 + tid; i < ph.R * 2; i += NTW) row_tab[i] = 0;
    }
}

// The same plan for launches of at most 64 sequences and 64 slots per kv head, worked out by every wave for itself with
// cross-lane operations (lane = sequence, then lane = row group): no LDS, no barriers.  (The general form below meets
// sixteen workgroup barriers; on four sequences it took 2.6 us of every workgroup's prologue.)
__device__ __forceinline__ int wave_scan_inclusive(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);    // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);    // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);    // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);    // row_shr:8: inclusive within rows of 16 lanes
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);    // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);    // row_bcast:31 into rows 2 and 3
    return v;
}
template <int NTW>
__device__ __forceinline__ PlanSlot plan_slot_wave(const PagedDevHeader& ph, int item, int hkv, int GQ, int T, int tid) {
    const int lane = tid & 63;
    const int pslots = ph.nitems;
    const int cap = ph.block_size * ph.max_blocks;
    // lane = sequence
    int qs = 0, qe = 0, tiles = 0, cnt = 0;
    if (lane < ph.W) {
        qs = min(max(ph.cu_q[lane], 0), T);
        qe = min(max(ph.cu_q[lane + 1], qs), T);
        int len = 0;
        for (int f = 0; f < ph.F; ++f) len = max(len, ph.frag_len[f * ph.W + lane]);
        len = min(len, cap);
        tiles = (len + TILE - 1) / TILE;
        cnt = ((qe - qs) * GQ + WIDE_ROWS - 1) / WIDE_ROWS;
    }
    const int gend = wave_scan_inclusive(cnt);          // row groups up to and including this sequence
    const int G = min(__builtin_amdgcn_readlane(gend, 63), min(64, pslots));
    // lane = row group: its sequence is the first whose groups reach beyond it
    int w = 0;
    for (int sq = 0; sq < ph.W; ++sq) w += __builtin_amdgcn_readlane(gend, sq) <= lane ? 1 : 0;
    w = min(w, ph.W - 1);
    const int w_gend = __shfl(gend, w, 64), w_cnt = __shfl(cnt, w, 64), w_qs = __shfl(qs, w, 64), w_qe = __shfl(qe, w, 64);
    const int w_tiles = __shfl(tiles, w, 64);
    const bool valid = lane < G;
    const int rg = lane - (w_gend - w_cnt);
    const int rows = min((w_qe - w_qs) * GQ - rg * WIDE_ROWS, WIDE_ROWS);
    const int work = valid ? w_tiles * (rows > WIDE_ROWS / 2 ? 4 : 3) : 0;
    const int most = max(1, w_tiles / 4);
    auto wave_total = [&](int v) { return __builtin_amdgcn_readlane(wave_scan_inclusive(v), 63); };
    // one slot each, and the other pslots - G in proportion to the work (see plan_slot)
    const int all_work = wave_total(work);
    const float share = (float)(pslots - G) * (1.0f - 1.0f / (1 << 20)) * __builtin_amdgcn_rcpf((float)max(all_work, 1));
    int n = valid ? min(1 + (int)((float)work * share), most) : 0;
    const int left = pslots - wave_total(n);
    const int load = (valid && n < most) ? __float_as_int((float)work * __builtin_amdgcn_rcpf((float)n)) : -1;
    int ahead = 0;
    for (int g = 0; g < G; ++g) {
        const int lg = __builtin_amdgcn_readlane(load, g);
        ahead += (lg > load || (lg == load && g < lane)) ? 1 : 0;
    }
    if (load >= 0 && ahead < left) ++n;
    const int slot0 = wave_scan_inclusive(n) - n;
    n = max(min(n, pslots - slot0), 0);                 // (cannot bite)
    const unsigned long long owner = __ballot(valid && item >= slot0 && item < slot0 + n);
    PlanSlot r;
    r.found = owner != 0;
    const int l = r.found ? __builtin_ctzll(owner) : 0;
    r.w = __builtin_amdgcn_readlane(w, l);
    r.rg = __builtin_amdgcn_readlane(rg, l);
    r.qs = __builtin_amdgcn_readlane(w_qs, l);
    r.qe = __builtin_amdgcn_readlane(w_qe, l);
    r.split = item - __builtin_amdgcn_readlane(slot0, l);
    r.ns = __builtin_amdgcn_readlane(n, l);
    plan_row_table<NTW>(ph, r, item, hkv, GQ, tid, __builtin_amdgcn_readlane(qe, ph.W - 1));
    return r;
}

template <int NTW>
__device__ __forceinline__ PlanSlot plan_slot(const PagedDevHeader& ph, int* lds, int item, int hkv, int GQ, int T, int tid) {
    constexpr int NT = PLAN_MAX_GROUPS;     // threads that take part (the others only meet the barriers)
    static_assert(NTW >= NT && WIDE_ROWS <= NT, "one thread per sequence, per row group, per row of a group");
    const bool act = tid < NT;
    int* sc_a = lds;                     // scan buffers
    int* sc_b = lds + NT;
    int* seq_qs = lds + 2 * NT;
    int* seq_qe = lds + 3 * NT;
    int* seq_tiles = lds + 4 * NT;
    int* grp_w = lds + 5 * NT;
    int* grp_rg = lds + 6 * NT;
    int* wave_part = lds + 7 * NT;       // [NTW / 64]
    int* shared = lds + 7 * NT + NTW / 64;        // total of a scan; then the slot's entry (6 ints)
    const int lane = tid & 63, wv = tid >> 6;
    const int pslots = ph.nitems;

    // Inclusive scan of one int per thread over the first `nact` threads (the others hold zero and get nothing useful
    // back); the sum of all goes to shared[0].
    auto scan = [&](int v, int nact) {
        int* src = sc_a;
        int* dst = sc_b;
        if (act) src[tid] = v;
        __syncthreads();
        for (int off = 1; off < nact; off <<= 1) {
            if (act) dst[tid] = src[tid] + (tid >= off ? src[tid - off] : 0);
            __syncthreads();
            int* t = src; src = dst; dst = t;
        }
        const int r = act ? src[tid] : 0;
        if (tid == nact - 1) shared[0] = r;
        __syncthreads();
        return r;
    };
    // Sum of one int per thread over the workgroup: DPP within rows of 16 lanes, the four rows of a wave by readlane, the
    // waves through LDS.
    auto block_total = [&](int v) {
        v += row_dpp<0xB1>(v);
        v += row_dpp<0x4E>(v);
        v += row_dpp<0x141>(v);
        v += row_dpp<0x140>(v);
        const int wt = __builtin_amdgcn_readlane(v, 0) + __builtin_amdgcn_readlane(v, 16) + __builtin_amdgcn_readlane(v, 32) +
                       __builtin_amdgcn_readlane(v, 48);
        if (lane == 0) wave_part[wv] = wt;
        __syncthreads();
        int s = wave_part[0];
#pragma unroll
        for (int i = 1; i < NTW / 64; ++i) s += wave_part[i];
        return s;
    };

    // sequences: query-token range, row groups, tiles of the KV any fragment may see
    const int cap = ph.block_size * ph.max_blocks;
    int cnt = 0;
    if (tid < ph.W) {
        const int qs = min(max(ph.cu_q[tid], 0), T);
        const int qe = min(max(ph.cu_q[tid + 1], qs), T);
        int len = 0;
        for (int f = 0; f < ph.F; ++f) len = max(len, ph.frag_len[f * ph.W + tid]);
        len = min(len, cap);
        seq_qs[tid] = qs;
        seq_qe[tid] = qe;
        seq_tiles[tid] = (len + TILE - 1) / TILE;
        cnt = ((qe - qs) * GQ + WIDE_ROWS - 1) / WIDE_ROWS;
    }
    const int gend = scan(cnt, ph.W);                   // row groups up to and including this sequence
    for (int g = gend - cnt; g < min(gend, NT); ++g) {  // (a malformed prefix array could ask for more groups than threads)
        grp_w[g] = tid;
        grp_rg[g] = g - (gend - cnt);
    }
    const int G = min(shared[0], min(NT, pslots));
    __syncthreads();

    // row groups: work, and the most slots it may take (four tiles per slot at least)
    int gw = 0, grg = 0, work = 0, most = 1, rows = 0;
    if (tid < G) {
        gw = grp_w[tid];
        grg = grp_rg[tid];
        rows = min((seq_qe[gw] - seq_qs[gw]) * GQ - grg * WIDE_ROWS, WIDE_ROWS);
        work = seq_tiles[gw] * (rows > WIDE_ROWS / 2 ? 4 : 3);
        most = max(1, seq_tiles[gw] / 4);
    }
    // One slot each, and the other pslots - G in proportion to the work (rounded down, so they fit; the quotient in
    // floating point, nudged down so that it never exceeds the exact one).
    const int all_work = block_total(work);
    const float share = (float)(pslots - G) * (1.0f - 1.0f / (1 << 20)) * __builtin_amdgcn_rcpf((float)max(all_work, 1));
    int n = tid < G ? min(1 + (int)((float)work * share), most) : 0;
    // what the rounding left over (fewer slots than groups) goes, one slot each, to the groups with the most work per slot
    const int left = pslots - block_total(n);
    const int load = (tid < G && n < most) ? __float_as_int((float)work * __builtin_amdgcn_rcpf((float)n)) : -1;   // (>= 0: ordered like the floats)
    if (act) sc_a[tid] = load;
    __syncthreads();
    int ahead = 0;
    for (int g = 0; g < G; ++g) ahead += (sc_a[g] > load || (sc_a[g] == load && g < tid)) ? 1 : 0;
    if (load >= 0 && ahead < left) ++n;
    __syncthreads();                                    // sc_a is a scan buffer again
    const int slot0 = scan(n, G) - n;
    n = max(min(n, pslots - slot0), 0);                 // (cannot bite)

    // the group that owns this workgroup's slot publishes the entry
    if (tid == 0) shared[1] = -1;
    __syncthreads();
    if (tid < G && item >= slot0 && item < slot0 + n) {
        shared[1] = gw; shared[2] = grg; shared[3] = seq_qs[gw]; shared[4] = seq_qe[gw]; shared[5] = item - slot0; shared[6] = n;
    }
    __syncthreads();
    PlanSlot r;
    r.w = shared[1]; r.rg = shared[2]; r.qs = shared[3]; r.qe = shared[4]; r.split = shared[5]; r.ns = shared[6];
    r.found = r.w >= 0;
    plan_row_table<NTW>(ph, r, item, hkv, GQ, tid, seq_qe[ph.W - 1]);
    return r;
}

// The paged operators (hogwild_paged_sdpa / hogwild_varlen_paged_sdpa, see hogwild_paged.hip) for many query rows per
// sequence: one workgroup = one kv head x one group of up to 128 rows of ONE sequence x every nsplit-th 32-token tile of
// that sequence, with the tile ring of attention_wide_kernel.  What differs is where a tile's rows lie: position l of
// sequence w is row l % block_size of block block_table[w][l / block_size] (src/kernels/kernel_v21.cuh:405-411).  The
// sequence's block table is copied into LDS once (up to PAGED_WIDE_MAX_BLOCKS entries; the launcher sends longer tables
// to the narrow kernel).  Per tile every lane derives the cache rows it fetches from it; positions no row of the group
// can see are redirected to the last visible one (no byte outside the visible part of the sequence is read; block ids
// are clamped into the cache).  NW waves: NW / PAR of them differ in their rows, and the PAR waves that share their rows
// take the tiles of a step in turn and add up their partial sums at the end (see PAGED_WIDE_WAVES).
template <class DT, int E, int EV, int NS, int NW, int PAR>
__global__ __launch_bounds__(NW * 64, 1) void paged_wide_kernel(const PagedHeader args) {

    typedef Geo<DT, E, EV> G;
    constexpr int NT = NW * 64;
    constexpr int NRW = NW / PAR;                // waves that differ in their rows; PAR waves share the rows and alternate on the tiles
    constexpr int RB = WIDE_ROWS / 16 / NRW;     // 16-row blocks per wave when the row group has more than 64 rows
    constexpr int TPR = NT / WIDE_ROWS;
    constexpr int NSTEP = NS / PAR;              // ring slots in steps of PAR tiles (one barrier per step)
    constexpr int DP = NSTEP - 1;                // steps requested ahead
    constexpr int KBYTES = G::KSTAGE;
    constexpr int VBYTES = TILE * G::VROW;
    constexpr int TPW = (KBYTES + VBYTES) / 1024 / NW;
    constexpr int TPS = PAR * TPW;               // transfers a wave issues per step
    constexpr int SLOT = KBYTES + VBYTES;
    constexpr int RPL = 64 / G::CPR;             // tile rows one transfer covers
    static_assert(G::SZ == 2 && KBYTES == VBYTES && TPW >= 1 && (2 * KBYTES / 1024) % TPW == 0 && NS % PAR == 0 && DP >= 1 && G::KROW == G::VROW &&
                      NW % PAR == 0 && (PAR == 1 || PAR == 2) && RB >= 1,
                  "16-bit types; a wave's transfers belong to one image");

    // The rotated queries are needed in LDS only until every wave holds its rows as MFMA operands: they lie behind the
    // ring slots that the first DP steps are requested into, in slots that are first requested into after the first
    // barrier of the tile loop.
    constexpr int QOFF = DP * PAR * SLOT;
    constexpr int QBYTES = WIDE_ROWS * G::QSTR;
    constexpr int RING_BYTES = NS * SLOT > QOFF + QBYTES ? NS * SLOT : QOFF + QBYTES;
    __shared__ int lim_lds[WIDE_ROWS];
    __shared__ int bt_lds[PAGED_WIDE_MAX_BLOCKS];
    __shared__ __attribute__((aligned(16))) char ring[RING_BYTES];
    char* const q_lds = ring + QOFF;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rw = wv % NRW;                     // which rows
    const int par = wv / NRW;                    // which tiles of a step
    const int n = lane & 15;
    const int q = lane >> 4;

    HW_MARK(8);
    PagedHeaderBits hb;
    paged_header_request(hb);
    // This wave's share of a tile's transfers.  With an even number of them a wave brings the same rows of both images:
    // a row of the K cache and the row of the V cache with the same number lie at the same place of their caches, so one
    // block look-up serves two transfers.  Otherwise the first half of the waves fill the K image, the second half V.
    constexpr bool BOTH = TPW % 2 == 0;
    constexpr int NI = BOTH ? 2 : 1;              // images a wave fills
    constexpr int NP = TPW / NI;                  // 1 KB pieces of each
    static_assert((KBYTES / 1024) % NP == 0 && NW * NP * NI * 1024 == KBYTES + VBYTES, "the waves' pieces tile both images");
    const bool k_wave = BOTH || wv < NW / 2;
    const int first = (BOTH ? wv : (k_wave ? wv : wv - NW / 2)) * NP;
    const int lrow = lane / G::CPR, lslot = lane % G::CPR;
    unsigned chunk[NI][NP];                       // byte offset of this lane's 16 bytes within its row, per image and piece
    int trow[NP];                                 // the tile row it belongs to
#pragma unroll
    for (int j = 0; j < NP; ++j) {
        const int row = (first + j) * RPL + lrow;
        const int key = G::CPR >= 16 ? (row & 15) : ((row >> 1) & (G::CPR - 1));
        const unsigned kchunk = (unsigned)((lslot ^ key) << 4), vchunk = (unsigned)((lslot ^ (2 * vimg_segment_key<G::VROW>(row))) << 4);
        trow[j] = row;
        chunk[0][j] = k_wave ? kchunk : vchunk;
        if constexpr (BOTH) chunk[1][j] = vchunk;
    }
    unsigned my_image[NI];                        // where the pieces go in ring slot 0
    my_image[0] = lds_address(ring) + (k_wave ? 0 : KBYTES) + first * 1024;
    if constexpr (BOTH) my_image[1] = my_image[0] + KBYTES;
    unsigned voff[G::NOC];                             // this lane's positions in a V image (transposed reads)
    vtr_lane_offsets<G::VROW>(voff, lane);
    const PagedDevHeader ph = paged_header_wait(hb);
    HW_MARK(0);

    // logical workgroup id = ((kv head * nitems) + item) * nsplit + split; consecutive ids share an XCD
    int bid = blockIdx.x;
    if (ph.flags & PH_XCD_REMAP) bid = (bid & 7) * (ph.nwg >> 3) + (bid >> 3);
    const int hi = fast_div(bid, ph.magic_nsplit);
    int split = bid - hi * ph.nsplit;
    const int hkv = fast_div(hi, ph.magic_nitems);
    const int item = hi - hkv * ph.nitems;
    const int GQ = ph.Hq / ph.Hkv;
    const int T = ph.LW * ph.LS;

    // Which rows of which sequence, and which share of its tiles.  A launch planned on the device (PH_PLANNED) says so in
    // the slot table behind the partial sums, one entry per workgroup slot of a kv head; otherwise the item is a row
    // group in the order of the sequences, every one with the same nsplit workgroups.
    int w, rg, qs, qe, ns;
    size_t pbase;                           // row of the partial arrays that holds the workgroup's first row
    if (ph.flags & PH_PLANNED) {
        const PlanSlot ps = (ph.W <= 64 && ph.nitems <= 64)      // uniform over the launch
                                ? plan_slot_wave<NT>(ph, item, hkv, GQ, T, tid)
                                : plan_slot<NT>(ph, reinterpret_cast<int*>(ring), item, hkv, GQ, T, tid);   // (the ring is not in use yet)
        if (!ps.found) return;              // a slot the plan left empty; uniform over the workgroup
        w = __builtin_amdgcn_readfirstlane(ps.w);
        rg = __builtin_amdgcn_readfirstlane(ps.rg);
        qs = __builtin_amdgcn_readfirstlane(ps.qs);
        qe = __builtin_amdgcn_readfirstlane(ps.qe);
        split = __builtin_amdgcn_readfirstlane(ps.split);
        ns = __builtin_amdgcn_readfirstlane(ps.ns);
        pbase = (size_t)(hkv * ph.nitems + item) * PLAN_SLOT_ROWS;
    } else {
        const PagedItem it = paged_item<WIDE_ROWS>(ph, item, lane, GQ);
        if (!it.found) return;              // the grid is sized for the worst case; uniform over the workgroup
        w = it.w, rg = it.rg, qs = it.qs, qe = it.qe;
        ns = ph.nsplit;
        pbase = (size_t)(hkv * ph.nsplit + split) * ph.R + (size_t)qs * GQ + (size_t)rg * WIDE_ROWS;
    }
    HW_MARK(6);
    HW_NOTE(9, (w << 20) | (rg << 12) | (split << 6) | ns);
    const int r0 = qs * GQ + rg * WIDE_ROWS;    // first row of the workgroup (global numbering: token * GQ + head in group)
    const int rend = qe * GQ;                   // end of the worker's rows
    if (r0 >= rend) return;                     // uniform over the workgroup
    const int cap = ph.block_size * ph.max_blocks;
    const HW_GLOBAL int* btw = ph.block_table + (size_t)w * ph.max_blocks;
    unsigned long long image[NI];
    image[0] = reinterpret_cast<unsigned long long>(k_wave ? ph.kcache : ph.vcache);
    if constexpr (BOTH) image[1] = reinterpret_cast<unsigned long long>(ph.vcache);

    DevHeader a;
    a.q = ph.q;
    a.loc = ph.loc;
    a.cos = nullptr;
    a.sin = nullptr;
    a.rq = nullptr;
    a.part_o = ph.part_o;
    a.part_ml = ph.part_ml;
    a.len_dev = nullptr;
    a.F = ph.F; a.W = ph.LW; a.Hq = ph.Hq; a.Hkv = ph.Hkv; a.S = ph.LS; a.R = rend;
    a.nrg = 1; a.wgs_per_head = ph.nsplit; a.nwg = ph.nwg;
    a.slot_stride = ph.nsplit; a.flags = KH_PREROTATED; a.sc = ph.sc;
    a.magic_gq = ph.magic_gq; a.magic_s = ph.magic_ls; a.magic_nrg = 0; a.magic_wg = 0;

    // The sequence's block table goes into LDS once: per tile every lane then looks up the block of its own position
    // there.  (Read from memory per tile it is either a vector load, which the hand-counted tile transfers would have
    // to wait behind, or a scalar load, whose latency every LDS wait of the tile loop then inherits: measured, 0.4 us
    // per tile.)
    {
        const int nent = min(ph.max_blocks, PAGED_WIDE_MAX_BLOCKS);
        for (int i = tid; i < nent; i += NT) bt_lds[i] = btw[i];
    }

    // (The rest as a function of the 16-row blocks per wave, RBX: two for row groups of more than 64 rows, one for the
    // others, behind one branch per workgroup.  With the branch inside the fragment loop instead, the two copies shared
    // their registers and the two-block tile loops ran 8 % slower.)
    auto run = [&](auto rbx) {
        constexpr int RBX = decltype(rbx)::value;
        constexpr int wrows = 16 * RBX;             // rows per wave
        const int w0 = r0 + rw * wrows;             // first row of this wave
        WaveState<RBX, G::NOC> st;
#pragma unroll
        for (int rb = 0; rb < RBX; ++rb) {
            st.m[rb] = NEG_BIG;
            st.l[rb] = 0.f;
#pragma unroll
            for (int c = 0; c < G::NOC; ++c) st.o[rb][c] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        st.fresh = true;

        for (int f = 0; f < ph.F; ++f) {
            // (the thread index as the compiler cannot see through it: what the prologue derives from it -- rows, addresses of
            // the queries -- is then formed here, per fragment, instead of once in front of the loop, from where it would stay
            // in registers across the tile loops, which have none to spare)
            int tidf = tid;
            asm volatile("" : "+v"(tidf));
            QueryRotation<DT, E, WIDE_ROWS, G::QSTR, true, NT> qrot;
            qrot.load(a, f, hkv, r0, GQ, tidf);
            const int lm = ph.loc[(size_t)f * T + fast_div(min(r0 + tidf / TPR, rend - 1), ph.magic_gq)];
            const int flen = ph.frag_len[ph.cu_q != nullptr ? f * ph.W + w : f];

            __syncthreads();   // the previous fragment's readers are done with q_lds / lim_lds / the ring
            if (f == 0) HW_MARK(7);
            qrot.finish(a, q_lds, f, hkv, r0, GQ, false, tidf);
            // (computed by every thread and pinned there: the compiler waits for a load where its result is first used, and a
            // use under the condition below leaves the wait to whatever next touches the registers -- inside the tile loops,
            // where a wait for "all loads" also waits for the look-ahead transfers it does not know of)
            int limv = (r0 + tidf / TPR < rend) ? max(0, min(min(flen, cap), lm < cap ? lm + 1 : cap)) : 0x7fffffff;
            asm volatile("" : "+v"(limv));
            if (tidf % TPR == 0) lim_lds[tidf / TPR] = limv;
            __syncthreads();
            if (f == 0) HW_MARK(1);

            {
                u32x4 qreg[RBX * G::KJ];
#pragma unroll
                for (int rb = 0; rb < RBX; ++rb)
#pragma unroll
                    for (int j = 0; j < G::KJ; ++j)
                        qreg[rb * G::KJ + j] = *reinterpret_cast<const u32x4*>(q_lds + (rw * wrows + rb * 16 + n) * G::QSTR + (4 * j + q) * 16);
                int lim[RBX];
                int maxlim = 0, minlim = 0x7fffffff;
#pragma unroll
                for (int rb = 0; rb < RBX; ++rb) {
                    lim[rb] = lim_lds[rw * wrows + rb * 16 + n];
                    const bool pad = w0 + rb * 16 + n >= rend;
                    maxlim = max(maxlim, pad ? 0 : lim[rb]);
                    minlim = min(minlim, lim[rb]);
                }
                maxlim = __builtin_amdgcn_readfirstlane(row_max16(maxlim));
                minlim = __builtin_amdgcn_readfirstlane(row_min16(minlim));
                // what the WORKGROUP can see decides which positions are fetched and where its tile loop ends (every wave must
                // take part in every step's barrier); what the wave can see decides which tiles it multiplies
                int wgmax = 0;
#pragma unroll
                for (int i = 0; i < WIDE_ROWS / 64; ++i) {
                    const int r = i * 64 + lane;
                    wgmax = max(wgmax, r0 + r < rend ? lim_lds[r] : 0);
                }
#pragma unroll
                for (int off = 1; off < 64; off <<= 1) wgmax = max(wgmax, __shfl_xor(wgmax, off, 64));
                wgmax = __builtin_amdgcn_readfirstlane(wgmax);

                // Source addresses of this wave's share of the PAR tiles of the step that starts at tile tb (TPS transfers):
                // every lane looks up the block of the row it fetches in each transfer.  A position beyond what the workgroup
                // can see is replaced by the last visible one, so a tile that does not exist costs the same number of
                // transfers and no new memory traffic to speak of, and no byte outside the visible part of the sequence is
                // read.
                auto addresses = [&](unsigned long long* src, int tb) {
#pragma unroll
                    for (int pp = 0; pp < PAR; ++pp)
#pragma unroll
                        for (int j = 0; j < NP; ++j) {
                            const int tok = min((tb + pp * ns) * TILE + trow[j], wgmax - 1);
                            const int bi = fast_div(tok, ph.magic_bs);
                            const int blk = min(max(bt_lds[bi], 0), ph.num_blocks - 1);
                            const int rid = (blk * ph.Hkv + hkv) * ph.block_size + (tok - bi * ph.block_size);
#pragma unroll
                            for (int im = 0; im < NI; ++im)
                                src[(pp * NP + j) * NI + im] = image[im] + (unsigned long long)(unsigned)rid * G::KROW + chunk[im][j];
                        }
                };
                auto request = [&](int step_slot, const unsigned long long* src) {
#pragma unroll
                    for (int pp = 0; pp < PAR; ++pp)
#pragma unroll
                        for (int j = 0; j < NP; ++j)
#pragma unroll
                            for (int im = 0; im < NI; ++im)
                                lds_transfer_flat(__builtin_amdgcn_readfirstlane(my_image[im] + (step_slot * PAR + pp) * SLOT + j * 1024),
                                                  src[(pp * NP + j) * NI + im]);
                };

                if (wgmax > 0) {   // uniform over the workgroup
                    // Tiles of this workgroup: split, split + ns, ...; a step is PAR of them, one for each of the waves that
                    // share their rows, behind one barrier.  The first DP steps are requested here; every later one right
                    // behind the barrier that frees its slots (all waves have left the step before), with addresses formed a
                    // step earlier, next to the arithmetic: a request is then TPS transfers and nothing else.
                    const int tstep = PAR * ns;
                    int first_tile = __builtin_amdgcn_readfirstlane(split);   // (opaque, like tidf: the positions of the first steps are formed here)
                    asm volatile("" : "+s"(first_tile));
                    unsigned long long src[TPS];
#pragma unroll
                    for (int i = 0; i < DP; ++i) {
                        addresses(src, first_tile + i * tstep);
                        request(i, src);
                    }
                    addresses(src, first_tile + DP * tstep);
                    // (the operands and bounds read out of LDS above have arrived before any wave passes the first barrier and
                    // requests into the slots the queries lie in)
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    // two loops with one instantiation of the tile arithmetic each (see attention_wide_kernel)
                    int sl = 0;                                   // step slot of the current step
                    int tb = first_tile;                          // its first tile
                    auto arrive = [&]() {
                        // this wave's transfers of the step have landed (the DP - 1 steps requested since may stay in flight:
                        // loads complete in order), then every wave's: a plain barrier, no fence that would wait for the
                        // look-ahead.  Behind it the slots of the step before are free: request step + DP into them.
                        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((DP - 1) * TPS) : "memory");
                        request(sl == 0 ? NSTEP - 1 : sl - 1, src);
                        addresses(src, tb + (DP + 1) * tstep);
                    };
                    const int tfast = maxlim > 0 ? min(minlim, wgmax) / TILE : 0;   // tiles below it are seen completely by every row of the wave
#pragma unroll 1
                    for (; tb + par * ns < tfast; tb += tstep) {
                        arrive();
                        const char* slot = ring + (sl * PAR + par) * SLOT;
                        compute_tile<DT, E, EV, RBX, false, true, false, true>(TileRegs<DT, E, EV>(), q_lds, qreg, lim, st, (tb + par * ns) * TILE, n, q, ph.sc, slot, slot + KBYTES, voff);
                        sl = sl + 1 == NSTEP ? 0 : sl + 1;
                    }
#pragma unroll 1
                    for (; tb * TILE < wgmax; tb += tstep) {      // uniform over the workgroup: every wave leaves at the same step
                        arrive();
                        if ((tb + par * ns) * TILE < maxlim) {
                            const char* slot = ring + (sl * PAR + par) * SLOT;
                            compute_tile<DT, E, EV, RBX, true, true, false, true>(TileRegs<DT, E, EV>(), q_lds, qreg, lim, st, (tb + par * ns) * TILE, n, q, ph.sc, slot, slot + KBYTES, voff);
                        }
                        sl = sl + 1 == NSTEP ? 0 : sl + 1;
                    }
                    // the requests behind the last tile must have landed before the ring is used again
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                }
            }
        }

        // ---- The PAR waves that share their rows hold a partial sum each: block rb of the rows goes to wave rb % PAR of
        // them through LDS (the ring, which no tile needs any more), lane for lane in the accumulator layout, and is
        // combined there.  Every wave then stores the blocks it owns, staged through LDS once more so that they leave as
        // whole rows (see attention_wide_kernel). ----
        {
            constexpr int OSTR = EV + 4;
            constexpr int REGION = 16 * OSTR;                     // floats per wave: a staged 16-row block, or a block in accumulator layout
            static_assert(G::NOC * 64 * 4 <= REGION && (NW * REGION + NW * 64 * 2) * 4 <= RING_BYTES, "the blocks of all waves fit into the ring");
            HW_MARK(3);
            __syncthreads();
            float* const regions = reinterpret_cast<float*>(ring);
            float* const mls = regions + NW * REGION;
            if constexpr (PAR > 1) {
#pragma unroll
                for (int rb = 0; rb < RBX; ++rb) {
                    const int owner = rw + (rb % PAR) * NRW;
                    if (owner != wv) {
#pragma unroll
                        for (int c = 0; c < G::NOC; ++c) *reinterpret_cast<f32x4*>(regions + owner * REGION + (c * 64 + lane) * 4) = st.o[rb][c];
                        *reinterpret_cast<f32x2*>(mls + (owner * 64 + lane) * 2) = f32x2{st.m[rb], st.l[rb]};
                    }
                }
                __syncthreads();
            }
            float* stage = regions + wv * REGION;
            {
#pragma unroll
                for (int rb = 0; rb < RBX; ++rb) {
                    if (rw + (rb % PAR) * NRW != wv) continue;    // uniform over the wave
                    if constexpr (PAR > 1) {
                        const f32x2 oml = *reinterpret_cast<const f32x2*>(mls + (wv * 64 + lane) * 2);
                        const float mnew = fmaxf(st.m[rb], oml.x);
                        const float mine = exp2f(st.m[rb] - mnew), theirs = exp2f(oml.x - mnew);
#pragma unroll
                        for (int c = 0; c < G::NOC; ++c) {
                            const f32x4 o2 = *reinterpret_cast<const f32x4*>(stage + (c * 64 + lane) * 4);
#pragma unroll
                            for (int i = 0; i < 4; ++i) st.o[rb][c][i] = st.o[rb][c][i] * mine + o2[i] * theirs;
                        }
                        st.l[rb] = st.l[rb] * mine + oml.y * theirs;
                        st.m[rb] = mnew;
                    }
                    const float lsum = quarter_sum(st.l[rb]);
                    const int row0 = w0 + rb * 16;
                    const size_t prow0 = pbase + (size_t)(row0 - r0);
#pragma unroll
                    for (int c = 0; c < G::NOC; ++c)              // block c, accumulator rows 4q .. 4q+3 = elements 16c + 4q ..
                        *reinterpret_cast<f32x4*>(stage + n * OSTR + 16 * c + 4 * q) = st.o[rb][c];
                    if (q == 0 && row0 + n < rend) *reinterpret_cast<HW_GLOBAL f32x2*>(ph.part_ml + (prow0 + n) * 2) = f32x2{st.m[rb], lsum};
                    const int nvalid = min(16, rend - row0);
                    HW_GLOBAL float* dst = ph.part_o + prow0 * EV;
#pragma unroll
                    for (int ps = 0; ps < 16 * EV / 256; ++ps) {
                        const int idx = ps * 256 + lane * 4;
                        const int rr = idx / EV, e = idx % EV;
                        if (rr < nvalid) *reinterpret_cast<HW_GLOBAL f32x4*>(dst + idx) = *reinterpret_cast<const f32x4*>(stage + rr * OSTR + e);
                    }
                }
            }
        }
        HW_MARK(5);
    };
    if (RB > 1 && rend - r0 <= WIDE_ROWS / 2) run(std::integral_constant<int, RB / 2>{});
    else run(std::integral_constant<int, RB>{});
}

// Waves per workgroup, how many of them share their rows, and ring slots (see PAGED_WIDE_WAVES for the layout).  On the
// multi-token benchmark workload (128 rows x 16 K tokens x 8 kv heads, fp16) four waves that take every tile measure the
// same with the same prologue (ring of 4 slots: 20.2-20.4 us against 20.3-20.8 us on one box): there the tile loop runs at
// the pace of the tile stream either way.
constexpr int WIDE_WAVES = 8;
constexpr int WIDE_PAR = 2;
constexpr int WIDE_SLOTS = 6;

template <class DT>
static hipError_t launch_wide_dt(const KernelArgs& ka, int E, hipStream_t stream) {
    constexpr int NS = WIDE_SLOTS;
    constexpr int NW = WIDE_WAVES;
    constexpr int PAR = WIDE_PAR;
    if (E != 64 && E != 128) return hipErrorInvalidValue;
    if (ka.h.flags & KH_PREROTATED) {
        if (E == 128) hipLaunchKernelGGL((attention_wide_kernel<DT, 128, 128, NS, true, NW, PAR>), dim3(ka.h.nwg), dim3(NW * 64), 0, stream, ka);
        else hipLaunchKernelGGL((attention_wide_kernel<DT, 64, 64, NS, true, NW, PAR>), dim3(ka.h.nwg), dim3(NW * 64), 0, stream, ka);
    } else {
        if (E == 128) hipLaunchKernelGGL((attention_wide_kernel<DT, 128, 128, NS, false, NW, PAR>), dim3(ka.h.nwg), dim3(NW * 64), 0, stream, ka);
        else hipLaunchKernelGGL((attention_wide_kernel<DT, 64, 64, NS, false, NW, PAR>), dim3(ka.h.nwg), dim3(NW * 64), 0, stream, ka);
    }
    return hipGetLastError();
}

hipError_t launch_attention_wide(const KernelArgs& ka, int dtype, int E, hipStream_t stream) {
    if (ka.h.len_dev != nullptr) return hipErrorInvalidValue;
    switch (dtype) {
        case 1: return launch_wide_dt<F16>(ka, E, stream);
        case 2: return launch_wide_dt<BF16>(ka, E, stream);
        default: return hipErrorInvalidValue;     // 16-bit types only
    }
}

// Waves per workgroup of the paged 128-row kernel: eight, two per SIMD.  The two waves of a SIMD share their rows (32
// rows = two 16-row blocks for a row group of more than 64 rows, else one block) and take every other tile: a step of the
// tile loop is two tiles behind one barrier, one for each of them.  So each wave reads half of the tiles out of LDS, and
// the arithmetic of one runs beside the waits of the other.  Measured on four 12 528-token sequences with 1/8/32/64,
// 1/1/1/64, 16 x 4, 64 x 4, 25 x 4 and 12 x 4 query tokens, against eight waves of 16 rows that all take every tile (which
// doubles what is read out of LDS per tile and row): 57.9 / 48.2 / 42.3 / 110.0 / 47.3 / 40.1 us against 64.7 / 52.4 / 43.4 /
// 116.4 / 50.6 / 39.2 us; that form had in turn been 4 % faster than four waves of 32 rows on every tile (one per SIMD).
// Ring of six 16 KB slots = three steps: one being multiplied, two in flight.  The two-block instantiation has to fit the
// 256 registers of a wave: a spill costs more than the registers it frees, because the compiler's wait for the reload
// also waits for the tile transfers in flight.
constexpr int PAGED_WIDE_WAVES = 8;
constexpr int PAGED_WIDE_PAR = 2;
constexpr int PAGED_WIDE_SLOTS = 6;

template <class DT>
static hipError_t launch_paged_wide_dt(const PagedHeader& ph, int E, hipStream_t stream) {
    constexpr int NS = PAGED_WIDE_SLOTS;
    constexpr int NW = PAGED_WIDE_WAVES;
    constexpr int PAR = PAGED_WIDE_PAR;
    if (E != 64 && E != 128) return hipErrorInvalidValue;
    if (E == 128) hipLaunchKernelGGL((paged_wide_kernel<DT, 128, 128, NS, NW, PAR>), dim3(ph.nwg), dim3(NW * 64), 0, stream, ph);
    else hipLaunchKernelGGL((paged_wide_kernel<DT, 64, 64, NS, NW, PAR>), dim3(ph.nwg), dim3(NW * 64), 0, stream, ph);
    return hipGetLastError();
}

hipError_t launch_paged_attention_wide(const PagedHeader& ph, int dtype, int E, hipStream_t stream) {
    if (ph.max_blocks > PAGED_WIDE_MAX_BLOCKS) return hipErrorInvalidValue;   // the table of a sequence must fit into LDS
    switch (dtype) {
        case 1: return launch_paged_wide_dt<F16>(ph, E, stream);
        case 2: return launch_paged_wide_dt<BF16>(ph, E, stream);
        default: return hipErrorInvalidValue;     // 16-bit types only
    }
}

}  // namespace hw

#ifdef HW_CLOCKS
extern "C" int hw_debug_read_wide_clocks(unsigned long long* host, size_t n) {
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(hw::hw_wide_clock_buf), n * sizeof(unsigned long long));
}
#endif

