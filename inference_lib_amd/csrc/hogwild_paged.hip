// Paged variants of the Hogwild! attention path for gfx950 (MI355X, CDNA4, wave64).
//
//   paged_attention_kernel ... the roles of hogwild_paged_attention_gpu_kernel21 (src/kernels/kernel_v21.cuh:318-602)
//                              and hogwild_varlen_paged_attention_gpu_kernel21 (:658-899) of the reference
//   copy_to_blocks_kernel .... copy_to_blocks_kernel (src/cache.cuh:6-49)
//
// The KV of worker (sequence) w lives in fixed-size blocks of one cache tensor, [num_blocks, Hkv, block_size, D],
// and position l of the sequence is found through block_table[w][l / block_size] (kernel_v21.cuh:405-411).
// Every "fragment" f attends the same sequence from position 0 with its own queries and its own bound
// min(fragment_lengths, location + 1) (kernel_v21.cuh:385-388).
//
// Work decomposition: a workgroup owns one kv head, one row group of one worker (up to 16 or 32 query rows, a row
// being one (token, q-head-in-group) pair of that worker) and every nsplit-th stripe of the sequence's 32-token
// tiles: tile t goes to wave t mod (4 * nsplit) of the (kv head, row group).  Nothing about the sequence lengths
// is known on the host (they are device tensors), so the stripes balance themselves.  The per-tile arithmetic,
// the LDS staging and the partial/merge scheme are those of the fragment kernel; what differs is the address
// generation: each lane computes the cache row of "its" token of the tile from the block table (one table entry
// per lane and tile, prefetched two tiles ahead), the rows a lane has to fetch are picked from those with
// ds_bpermute, and K goes global -> LDS / V global -> registers with per-lane 64-bit addresses.  Tokens that no
// row of the group can see are redirected to the last visible token, so no byte outside the visible part of the
// sequence is ever read; block ids are clamped into the cache, so a corrupt table cannot fault the GPU.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hogwild_kernels.h"
#include "hogwild_device.h"

// waves per SIMD the one-row-block 16-bit kernels are register-budgeted for (tuning knob)
#ifndef HW_PAGED_MINW
#define HW_PAGED_MINW 1
#endif

namespace hw {

template <class DT, int E, int EV, int RB, int MINW>
__global__ __launch_bounds__(NTHREADS, MINW) void paged_attention_kernel(const PagedHeader args) {
    typedef Geo<DT, E, EV> G;
    constexpr int ROWS = RB * 16;
    typedef hw::Exchange<ROWS, EV> Ex;
    constexpr int SBYTES = NWAVES * G::KSTAGE;
    __shared__ __attribute__((aligned(16))) char q_lds[ROWS * G::QSTR];
    __shared__ int lim_lds[ROWS];
    union Slot0 {
        char k[SBYTES];
        Ex ex;
    };
    __shared__ __attribute__((aligned(16))) Slot0 slot0;
    __shared__ __attribute__((aligned(16))) char slot1[SBYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int q = lane >> 4;
    char* const kslots[2] = {slot0.k + wv * G::KSTAGE, slot1 + wv * G::KSTAGE};

    PagedHeaderBits hb;
    paged_header_request(hb);
    // argument-independent setup while the header is in flight
    // K load i of a wave covers tile rows i*RPL .. i*RPL+RPL-1; this lane fetches a chunk of row i*RPL + lrow, and
    // which chunk follows from the bank swizzle, applied on the global side (the transfer writes LDS linearly)
    constexpr int RPL = 64 / G::CPR;
    const int lrow = lane / G::CPR, lslot = lane % G::CPR;
    auto k_chunk = [&](int i) -> unsigned {
        const int row = i * RPL + lrow;
        const int key = G::CPR >= 16 ? (row & 15) : ((row >> 1) & (G::CPR - 1));
        return (unsigned)((lslot ^ key) << 4);
    };
    WaveState<RB, G::NOC> st;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        st.m[rb] = NEG_BIG;
        st.l[rb] = 0.f;
#pragma unroll
        for (int c = 0; c < G::NOC; ++c) st.o[rb][c] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    st.fresh = true;
    const PagedDevHeader ph = paged_header_wait(hb);

    // logical workgroup id = ((kv head * nitems) + item) * nsplit + split; consecutive ids share an XCD
    int bid = blockIdx.x;
    if (ph.flags & PH_XCD_REMAP) bid = (bid & 7) * (ph.nwg >> 3) + (bid >> 3);
    const int hi = fast_div(bid, ph.magic_nsplit);
    const int split = bid - hi * ph.nsplit;
    const int hkv = fast_div(hi, ph.magic_nitems);
    const int item = hi - hkv * ph.nitems;
    const int GQ = ph.Hq / ph.Hkv;

    const PagedItem it = paged_item<ROWS>(ph, item, lane, GQ);
    if (!it.found) return;                  // the grid is sized for the worst case; uniform over the workgroup
    const int w = it.w, rg = it.rg, qs = it.qs, qe = it.qe;
    const int T = ph.LW * ph.LS;
    const int r0 = qs * GQ + rg * ROWS;     // first row (global numbering: token * GQ + head in group)
    const int rend = qe * GQ;               // end of the worker's rows
    if (r0 >= rend) return;                 // uniform over the workgroup
    const int cap = ph.block_size * ph.max_blocks;
    const int NW = ph.nsplit * NWAVES;      // waves that share the tiles of this (kv head, row group)
    const int gw = split * NWAVES + wv;
    const HW_GLOBAL int* btw = ph.block_table + (size_t)w * ph.max_blocks;

    // what QueryRotation / map_row need, in the [LW, Hq, LS] layout, with the worker's row end as the row limit
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

    // block-table entry of the token this lane stands for in tile t
    auto bt_load = [&](int t) -> int {
        const int tok = min(t * TILE + (lane & 31), cap - 1);
        return btw[fast_div(tok, ph.magic_bs)];
    };

    for (int f = 0; f < ph.F; ++f) {
        // one batch of independent loads: queries, locations, fragment length, the table entries of two tiles
        QueryRotation<DT, E, ROWS, G::QSTR, true> qrot;
        qrot.load(a, f, hkv, r0, GQ, tid);
        const int lm = ph.loc[(size_t)f * T + fast_div(min(r0 + (tid & (ROWS - 1)), rend - 1), ph.magic_gq)];
        const int flen = ph.frag_len[ph.cu_q != nullptr ? f * ph.W + w : f];
        int bt_a = bt_load(gw);
        int bt_b = bt_load(gw + NW);

        __syncthreads();   // the previous fragment's readers are done with q_lds / lim_lds
        qrot.finish(a, q_lds, f, hkv, r0, GQ, false, tid);
        if (tid < ROWS) lim_lds[tid] = (r0 + tid < rend) ? max(0, min(min(flen, cap), lm < cap ? lm + 1 : cap)) : 0x7fffffff;
        __syncthreads();

        constexpr bool QREG = MINW == 1;
        u32x4 qreg[QREG ? RB * G::KJ : 1];
        if constexpr (QREG) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int j = 0; j < G::KJ; ++j)
                    qreg[rb * G::KJ + j] = *reinterpret_cast<const u32x4*>(q_lds + (rb * 16 + n) * G::QSTR + (4 * j + q) * 16);
        }
        int lim[RB];
        int maxlim = 0, minlim = 0x7fffffff;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            lim[rb] = lim_lds[rb * 16 + n];
            const bool pad = r0 + rb * 16 + n >= rend;
            maxlim = max(maxlim, pad ? 0 : lim[rb]);
            minlim = min(minlim, lim[rb]);
        }
        maxlim = __builtin_amdgcn_readfirstlane(row_max16(maxlim));
        minlim = __builtin_amdgcn_readfirstlane(row_min16(minlim));

        // Issue the loads of tile t given its table entries: the same number of load instructions whether or not
        // the tile exists (a tile beyond the visible range re-reads one row that is visible, or, if nothing is
        // visible at all, some row inside the cache: a few hundred bytes that are never used).
        auto issue_tile = [&](TileRegs<DT, E, EV>& tr, char* kslot, int btv, int t) {
            const int tok_raw = t * TILE + (lane & 31);
            const int tok = min(tok_raw, cap - 1);
            const int bi = fast_div(tok, ph.magic_bs);
            const int blk = min(max(btv, 0), ph.num_blocks - 1);
            int rid = (blk * ph.Hkv + hkv) * ph.block_size + (tok - bi * ph.block_size);
            const int jstar = min(max(maxlim - 1 - t * TILE, 0), 31);
            const int rstar = __builtin_amdgcn_readlane(rid, jstar);
            rid = tok_raw < maxlim ? rid : rstar;
            asm volatile("" ::: "memory");   // the transfers keep their place between the reads of the slot (see load_tile)
#pragma unroll
            for (int i = 0; i < G::KL; ++i) {
                const int r = __shfl(rid, i * RPL + lrow, 64);
                const HW_GLOBAL char* src = ph.kcache + (unsigned long long)(unsigned)r * G::KROW + k_chunk(i);
                __builtin_amdgcn_global_load_lds(src, HW_LDS_PTR(kslot + i * 1024), 16, 0, HW_KV_AUX);
            }
            asm volatile("" ::: "memory");
#pragma unroll
            for (int idx = 0; idx < 8; ++idx) {
                const int r = __shfl(rid, slot_token(q, idx), 64);
                const HW_GLOBAL char* src = ph.vcache + (unsigned long long)(unsigned)r * G::VROW + n * (G::VLD * 4);
#pragma unroll
                for (int hh = 0; hh < G::NVL; ++hh) {
                    if constexpr (G::VLD == 4) {
                        const u32x4 x = HW_KV_AUX == 2 ? __builtin_nontemporal_load(reinterpret_cast<const HW_GLOBAL u32x4*>(src + hh * 256))
                                                        : *reinterpret_cast<const HW_GLOBAL u32x4*>(src + hh * 256);
                        tr.v[idx][hh * 4 + 0] = x.x;
                        tr.v[idx][hh * 4 + 1] = x.y;
                        tr.v[idx][hh * 4 + 2] = x.z;
                        tr.v[idx][hh * 4 + 3] = x.w;
                    } else {
                        const u32x2 x = HW_KV_AUX == 2 ? __builtin_nontemporal_load(reinterpret_cast<const HW_GLOBAL u32x2*>(src))
                                                        : *reinterpret_cast<const HW_GLOBAL u32x2*>(src);
                        tr.v[idx][0] = x.x;
                        tr.v[idx][1] = x.y;
                    }
                }
            }
        };

        if (maxlim > 0) {   // uniform
            // Two tiles in flight per wave.  Per step: request the table entries two tiles ahead, then the K/V of
            // the next tile (its entries were requested one step earlier, ahead of the previous K/V request, so
            // they have arrived by the time the current tile's data has), then compute the current tile.
            TileRegs<DT, E, EV> tr[2];
            issue_tile(tr[0], kslots[0], bt_a, gw);
            // Two loops with one instantiation of the tile arithmetic each (see attention_kernel): pairs of tiles every
            // row of the wave sees completely, then the rest.
            int t = gw;
            if constexpr (G::SZ != 4)               // (the fp32 kernels keep one loop with both instantiations, see attention_kernel)
            for (; (t + NW + 1) * TILE <= minlim; t += 2 * NW) {
                {
                    const int bt_n = bt_load(t + 2 * NW);
                    issue_tile(tr[1], kslots[1], bt_b, t + NW);
                    if constexpr (E > 128) wait_k_landed<G, 1>();   // (see wait_k_landed: the table load in between only adds to what is behind)
                    compute_tile<DT, E, EV, RB, false, QREG>(tr[0], q_lds, qreg, lim, st, t * TILE, n, q, ph.sc, kslots[0]);
                    bt_a = bt_n;
                }
                {
                    const int bt_n = bt_load(t + 3 * NW);
                    issue_tile(tr[0], kslots[0], bt_a, t + 2 * NW);
                    if constexpr (E > 128) wait_k_landed<G, 1>();
                    compute_tile<DT, E, EV, RB, false, QREG>(tr[1], q_lds, qreg, lim, st, (t + NW) * TILE, n, q, ph.sc, kslots[1]);
                    bt_b = bt_n;
                }
            }
            for (; t * TILE < maxlim; t += 2 * NW) {
                {
                    const int bt_n = bt_load(t + 2 * NW);
                    issue_tile(tr[1], kslots[1], bt_b, t + NW);
                    if constexpr (E > 128) wait_k_landed<G, 1>();
                    const int t0 = t * TILE;
                    if (G::SZ == 4 && t0 + TILE <= minlim) compute_tile<DT, E, EV, RB, false, QREG>(tr[0], q_lds, qreg, lim, st, t0, n, q, ph.sc, kslots[0]);
                    else compute_tile<DT, E, EV, RB, true, QREG>(tr[0], q_lds, qreg, lim, st, t0, n, q, ph.sc, kslots[0]);
                    bt_a = bt_n;
                }
                {
                    const int bt_n = bt_load(t + 3 * NW);
                    issue_tile(tr[0], kslots[0], bt_a, t + 2 * NW);
                    if constexpr (E > 128) wait_k_landed<G, 1>();
                    const int t0 = (t + NW) * TILE;
                    if (G::SZ == 4 && t0 + TILE <= minlim) compute_tile<DT, E, EV, RB, false, QREG>(tr[1], q_lds, qreg, lim, st, t0, n, q, ph.sc, kslots[1]);
                    else if (t0 < maxlim) compute_tile<DT, E, EV, RB, true, QREG>(tr[1], q_lds, qreg, lim, st, t0, n, q, ph.sc, kslots[1]);
                    bt_b = bt_n;
                }
            }
        }
    }

    store_partials<DT, EV, RB, true>(st, slot0.ex, wv, n, q, tid, ph.part_o, ph.part_ml, (size_t)(hkv * ph.nsplit + split) * ph.R + r0,
                               min(ROWS, rend - r0));
}

// Scatter of new K/V rows into the paged caches, one 16-byte chunk (or, for odd sizes, one element) per thread.
// A position whose block index lies outside the table, or whose table entry lies outside the cache, is skipped.
template <int VEC>   // bytes per thread
__global__ __launch_bounds__(256) void copy_to_blocks_kernel(const CopyBlocksArgs a, int sz) {
    const int ck = a.E * sz / VEC, cv = a.Ev * sz / VEC;
    const size_t rows = (size_t)a.B * a.Hkv * a.S_new;
    const size_t total = rows * (size_t)(ck + cv);
    for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
        const size_t row = idx / (size_t)(ck + cv);
        const int c = (int)(idx - row * (size_t)(ck + cv));
        const int t = (int)(row % a.S_new);
        const size_t bh = row / a.S_new;
        const int h = (int)(bh % a.Hkv);
        const int b = (int)(bh / a.Hkv);
        const long long pos = (long long)a.seq_lengths[b] + t;
        if (pos < 0) continue;
        const long long bi = pos / a.block_size;
        if (bi >= a.max_blocks) continue;
        const int blk = a.block_table[(size_t)b * a.max_blocks + bi];
        if (blk < 0 || blk >= a.num_blocks) continue;
        const int off = (int)(pos - bi * a.block_size);
        const size_t dst_row = ((size_t)blk * a.Hkv + h) * a.block_size + off;
        const bool is_k = c < ck;
        const char* src = is_k ? reinterpret_cast<const char*>(a.key_states) + ((long long)b * a.ks_b + (long long)h * a.ks_h + (long long)t * a.ks_s) * sz + (size_t)c * VEC
                               : reinterpret_cast<const char*>(a.value_states) + ((long long)b * a.vs_b + (long long)h * a.vs_h + (long long)t * a.vs_s) * sz + (size_t)(c - ck) * VEC;
        char* dst = is_k ? reinterpret_cast<char*>(a.kcache) + dst_row * a.E * sz + (size_t)c * VEC
                         : reinterpret_cast<char*>(a.vcache) + dst_row * a.Ev * sz + (size_t)(c - ck) * VEC;
        if constexpr (VEC == 16) *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(src);
        else if constexpr (VEC == 4) *reinterpret_cast<u32*>(dst) = *reinterpret_cast<const u32*>(src);
        else *reinterpret_cast<unsigned short*>(dst) = *reinterpret_cast<const unsigned short*>(src);
    }
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
template <class DT, int E, int EV>
static hipError_t launch_paged_rb(const PagedHeader& ph, int rb, hipStream_t stream) {
    constexpr bool half = Elem<DT>::size == 2;
    // fp32 operands with two row blocks do not fit the register file; the planner never asks for them
    if constexpr (half) {
        if (rb == 2) {
            hipLaunchKernelGGL((paged_attention_kernel<DT, E, EV, 2, 1>), dim3(ph.nwg), dim3(NTHREADS), 0, stream, ph);
            return hipGetLastError();
        }
    }
    if (rb != 1) return hipErrorInvalidValue;
    hipLaunchKernelGGL((paged_attention_kernel<DT, E, EV, 1, half ? HW_PAGED_MINW : 1>), dim3(ph.nwg), dim3(NTHREADS), 0, stream, ph);
    return hipGetLastError();
}

template <class DT>
static hipError_t launch_paged_dt(const PagedHeader& ph, int E, int rb, hipStream_t stream) {
    if (E == 256) {     // one 16-row block per workgroup, one wave per SIMD; 16-bit types (two fp32 K tiles per wave exceed the LDS)
        if constexpr (Elem<DT>::size == 2) {
            if (rb != 1) return hipErrorInvalidValue;
            hipLaunchKernelGGL((paged_attention_kernel<DT, 256, 256, 1, 1>), dim3(ph.nwg), dim3(NTHREADS), 0, stream, ph);
            return hipGetLastError();
        }
        return hipErrorInvalidValue;
    }
    if (E == 128) return launch_paged_rb<DT, 128, 128>(ph, rb, stream);
    if (E != 64) return hipErrorInvalidValue;
    return launch_paged_rb<DT, 64, 64>(ph, rb, stream);
}

hipError_t launch_paged_attention(const PagedHeader& ph, int dtype, int E, int rb, hipStream_t stream) {
    switch (dtype) {
        case 0: return launch_paged_dt<F32>(ph, E, rb, stream);
        case 1: return launch_paged_dt<F16>(ph, E, rb, stream);
        default: return launch_paged_dt<BF16>(ph, E, rb, stream);
    }
}

hipError_t launch_copy_to_blocks(const CopyBlocksArgs& ca, int dtype, hipStream_t stream) {
    const int sz = dtype == 0 ? 4 : 2;
    const bool vec16 = (ca.E * sz) % 16 == 0 && (ca.Ev * sz) % 16 == 0 && (ca.ks_b * sz) % 16 == 0 && (ca.ks_h * sz) % 16 == 0 &&
                       (ca.ks_s * sz) % 16 == 0 && (ca.vs_b * sz) % 16 == 0 && (ca.vs_h * sz) % 16 == 0 && (ca.vs_s * sz) % 16 == 0 &&
                       ((reinterpret_cast<uintptr_t>(ca.key_states) | reinterpret_cast<uintptr_t>(ca.value_states) |
                         reinterpret_cast<uintptr_t>(ca.kcache) | reinterpret_cast<uintptr_t>(ca.vcache)) & 15u) == 0;
    const int vec = vec16 ? 16 : sz;
    const size_t total = (size_t)ca.B * ca.Hkv * ca.S_new * (size_t)((ca.E + ca.Ev) * sz / vec);
    if (total == 0) return hipSuccess;
    size_t blocks = (total + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    if (vec == 16) hipLaunchKernelGGL((copy_to_blocks_kernel<16>), dim3((unsigned)blocks), dim3(256), 0, stream, ca, sz);
    else if (vec == 4) hipLaunchKernelGGL((copy_to_blocks_kernel<4>), dim3((unsigned)blocks), dim3(256), 0, stream, ca, sz);
    else hipLaunchKernelGGL((copy_to_blocks_kernel<2>), dim3((unsigned)blocks), dim3(256), 0, stream, ca, sz);
    return hipGetLastError();
}

}  // namespace hw
