// Device-side building blocks shared by the attention kernels of this library (gfx950, wave64): element traits,
// tile geometry, K/V tile loads, the per-tile MFMA + online-softmax step, query staging.  Included by the .hip
// translation units only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hogwild_kernels.h"

#ifndef HW_MARK
#define HW_MARK(i) do { } while (0)
#endif
// Cache-policy bits of the K/V tile loads: 2 = non-temporal.  Every K/V byte is used exactly once per launch, so
// the tiles are streamed past the caches instead of displacing the queries, tables and split-K partials
// (measured: 17.35 -> 15.6 us per decode step at the 51 MB workload).
constexpr int HW_KV_AUX = 2;

namespace hw {

typedef unsigned int u32;
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

struct BF16 {};
struct F16 {};
struct F32 {};

template <class DT> struct Elem;
template <> struct Elem<BF16> {
    typedef unsigned short store_t;
    static constexpr int size = 2;
    static __device__ __forceinline__ float to_float(store_t x) { return __uint_as_float(((u32)x) << 16); }
    static __device__ __forceinline__ store_t from_float(float f) {
        __bf16 h = (__bf16)f;
        return __builtin_bit_cast(unsigned short, h);
    }
    static __device__ __forceinline__ u32 pack2(float a, float b) {
        f32x2 v = {a, b};
        return __builtin_bit_cast(u32, __builtin_convertvector(v, bf16x2));
    }
    static __device__ __forceinline__ float dot(u32 a, u32 b, float c) {   // two elements per dword
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
    }
    static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Elem<F16> {
    typedef unsigned short store_t;
    static constexpr int size = 2;
    static __device__ __forceinline__ float to_float(store_t x) { return (float)__builtin_bit_cast(_Float16, x); }
    static __device__ __forceinline__ store_t from_float(float f) {
        _Float16 h = (_Float16)f;
        return __builtin_bit_cast(unsigned short, h);
    }
    static __device__ __forceinline__ u32 pack2(float a, float b) {
        f32x2 v = {a, b};
        return __builtin_bit_cast(u32, __builtin_convertvector(v, f16x2));
    }
    static __device__ __forceinline__ float dot(u32 a, u32 b, float c) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
    }
    static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};
template <> struct Elem<F32> {
    typedef float store_t;
    static constexpr int size = 4;
    static __device__ __forceinline__ float to_float(store_t x) { return x; }
    static __device__ __forceinline__ store_t from_float(float f) { return f; }
    static __device__ __forceinline__ float dot(u32 a, u32 b, float c) { return __builtin_fmaf(__uint_as_float(a), __uint_as_float(b), c); }
};

constexpr float NEG_BIG = -1.0e30f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Workgroup barrier for data exchanged through LDS only: waits for this wave's LDS operations, not for its outstanding
// global loads and global->LDS transfers.  (__syncthreads() carries a release fence, and the compiler makes every
// transfer into LDS issued before it land first: a K/V tile in flight would be drained at every barrier.)
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Reductions over the four lanes {l, l^16, l^32, l^48}: the four quarter-waves hold different tokens of one row.
// v_permlane32_swap / v_permlane16_swap exchange half-waves / 16-lane rows between two registers; applied to two
// copies of a value they leave "mine" in one register and "my partner's" in the other, in every lane, without the
// trip through the LDS crossbar that a generic shuffle takes.
__device__ __forceinline__ void quarter_pairs(float v, int step, float& a, float& b) {
    const u32 x = __float_as_uint(v);
    if (step == 32) {
        const auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
        a = __uint_as_float(r[0]);
        b = __uint_as_float(r[1]);
    } else {
        const auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);
        a = __uint_as_float(r[0]);
        b = __uint_as_float(r[1]);
    }
}
// max of two values that are never NaN.  fmaxf() on the halves of a lane exchange makes the compiler canonicalise both
// inputs first (v_max_f32 x, x, x: two extra instructions per maximum, 8 per tile); the instruction itself needs none.
__device__ __forceinline__ float max_nn(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float quarter_max(float v) {
    float a, b;
    quarter_pairs(v, 32, a, b);
    v = max_nn(a, b);
    quarter_pairs(v, 16, a, b);
    return max_nn(a, b);
}
__device__ __forceinline__ float quarter_sum(float v) {
    float a, b;
    quarter_pairs(v, 32, a, b);
    v = a + b;
    quarter_pairs(v, 16, a, b);
    return a + b;
}

// Maximum / minimum over the 16 lanes of a row (lane % 16 = query row; the four rows of a wave hold the same values) by
// four data-parallel-primitive moves: the two lane swaps within a quad, then the mirrored half row and the mirrored row.
// (A generic shuffle goes through the LDS crossbar: four dependent round trips instead.)
template <int CTRL>
__device__ __forceinline__ int row_dpp(int v) { return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xf, 0xf, false); }
__device__ __forceinline__ int row_max16(int v) {
    v = max(v, row_dpp<0xB1>(v));     // quad_perm [1,0,3,2]
    v = max(v, row_dpp<0x4E>(v));     // quad_perm [2,3,0,1]
    v = max(v, row_dpp<0x141>(v));    // row_half_mirror
    return max(v, row_dpp<0x140>(v)); // row_mirror
}
__device__ __forceinline__ int row_min16(int v) {
    v = min(v, row_dpp<0xB1>(v));
    v = min(v, row_dpp<0x4E>(v));
    v = min(v, row_dpp<0x141>(v));
    return min(v, row_dpp<0x140>(v));
}

// token (relative to the tile start) held in reduction slot `idx` (0..7) of quarter-wave `q`:
// slots 0..3 come from the first 16-token S^T block, 4..7 from the second (accumulator rows 4q..4q+3).
__device__ __forceinline__ int slot_token(int q, int idx) { return ((idx >> 2) << 4) + (q << 2) + (idx & 3); }

template <class DT, int E, int EV>
struct Geo {
    static constexpr int SZ = Elem<DT>::size;
    static constexpr int KJ = E * SZ / 64;               // 16-byte K operand chunks per lane per 16-token block
    static constexpr int KROW = E * SZ;                  // bytes of one K row
    static constexpr int VROW = EV * SZ;                 // bytes of one V row
    static constexpr int CPR = KROW / 16;                // 16-byte chunks per K row
    static constexpr int KL = TILE * KROW / 1024;        // 1 KB wave-wide K loads per tile
    static constexpr int KSTAGE = TILE * KROW;           // bytes of the per-wave K staging area in LDS
    static constexpr int VW = EV * SZ / 64;              // dwords of one V row held by one lane
    static constexpr int VLD = VW < 4 ? VW : 4;          // dwords per V load
    static constexpr int NVL = VW / VLD;                 // V loads per row per lane
    static constexpr int NOC = EV / 16;                  // 16-wide output chunks (accumulators per row block)
    static constexpr int QSTR = E * SZ + 16;             // LDS row stride of the rotated query (bytes)
};

// Registers of one 32-token tile of one wave: only V lives in registers, K goes straight from global memory
// into the wave's LDS staging slot.
template <class DT, int E, int EV>
struct TileRegs {
    typedef Geo<DT, E, EV> G;
    u32 v[8][G::VW];     // V rows of the lane's 8 reduction slots, VW dwords of each
};

#define HW_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define HW_GLOBAL __attribute__((address_space(1)))

// A fragment's K and V slices of one kv head.  K goes through a buffer resource: out-of-range rows read as zero, so
// its global->LDS transfers need no address clamping and a tile that does not exist costs no memory traffic.  V is
// read with plain global loads (measured: a tile's rows land ~15 % sooner than through buffer loads), with rows beyond
// the fragment redirected to its last row.
struct FragView {
    __amdgpu_buffer_rsrc_t k;
    unsigned long long vbase;   // start of the kv head's V rows
    unsigned long long idle;    // where the V loads of a tile that does not exist go: a line every workgroup keeps hot
    int L;
};
constexpr unsigned OOB_OFFSET = 0xFFFF0000u;   // beyond any fragment (lengths are validated on the host)

__device__ __forceinline__ FragView make_view(unsigned long long kptr, unsigned long long vptr, int hkv, int L, int cap, int krow, int vrow,
                                              unsigned long long idle) {
    FragView fv;
    fv.idle = idle;
    fv.k = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(kptr + (unsigned long long)hkv * cap * krow), 0, L * krow, 0x00020000);
    fv.vbase = vptr + (unsigned long long)hkv * cap * vrow;
    fv.L = L;
    return fv;
}

// LDS position of 16-byte chunk c of tile row `row` in a K staging slot.  The xor key makes the operand read
// (16 lanes = 16 different rows, same chunk) touch 16 different 16-byte bank groups.
template <class G>
__device__ __forceinline__ int kstage_offset(int row, int c) {
    const int key = G::CPR >= 16 ? (row & 15) : ((row >> 1) & (G::CPR - 1));
    return row * G::KROW + ((c ^ key) << 4);
}

// Per-lane byte offsets (within a tile) of the K chunk each lane fetches in each of the KL wave-wide loads.
// A load writes LDS linearly (lane l -> slot base + 16 l), so the bank swizzle of kstage_offset is applied on
// the global side: the lane that fills position (row, slot) fetches chunk slot ^ key(row) of that row.  The 16
// lanes of a row still cover the row's bytes exactly once, so every load remains 1 KB of whole rows.
template <class G>
__device__ __forceinline__ void k_lane_offsets(unsigned* koff, int lane) {
#pragma unroll
    for (int i = 0; i < G::KL; ++i) {
        const int p = i * 64 + lane;
        const int row = p / G::CPR, slot = p % G::CPR;
        const int key = G::CPR >= 16 ? (row & 15) : ((row >> 1) & (G::CPR - 1));
        koff[i] = row * G::KROW + ((slot ^ key) << 4);
    }
}

// Issue the loads of one tile: K by direct global->LDS transfers into `kslot` (this wave's part of a staging
// slot), V into registers.  The number of load instructions is the same whether or not the tile exists, which
// keeps the hardware wait counts exact on every path; a tile that does not exist costs (almost) no memory traffic.
template <class DT, int E, int EV>
__device__ __forceinline__ void load_tile(TileRegs<DT, E, EV>& t, const FragView& fv, char* kslot, const unsigned* koff, int t0,
                                          int n, int q, bool real) {
    typedef Geo<DT, E, EV> G;
    const unsigned kb = real ? (unsigned)(t0 * G::KROW) : OOB_OFFSET;
    // The transfers keep their place in program order: behind every earlier read of the slot and ahead of everything
    // that follows.  (The compiler models a transfer as a 16-byte store at its LDS base, not as the 1 KB it is, and has
    // moved operand reads of the same slot in between the transfers of a tile on the strength of that.)
    asm volatile("" ::: "memory");
#pragma unroll
    for (int i = 0; i < G::KL; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(fv.k, HW_LDS_PTR(kslot + i * 1024), 16, kb + koff[i], 0, 0, HW_KV_AUX);
    asm volatile("" ::: "memory");
    // V: a quarter-wave reads one whole row (or half of a 512-byte row) per load.  Rows beyond the fragment are
    // redirected to its last row (their probabilities are zero); a tile that does not exist reads one cached line
    // (fv.idle) with every lane: loads return in order, so what such a load costs is its own latency behind the last
    // real tile, and that must be a cache hit, not a trip to memory.
#pragma unroll
    for (int idx = 0; idx < 8; ++idx) {
        const int row = min(t0 + q * 4 + (idx >> 2) * 16 + (idx & 3), fv.L - 1);
        const unsigned long long addr = real ? fv.vbase + (unsigned long long)(unsigned)row * G::VROW + n * (G::VLD * 4) : fv.idle;
#pragma unroll
        for (int hh = 0; hh < G::NVL; ++hh) {
            if constexpr (G::VLD == 4) {
                const u32x4 x = __builtin_nontemporal_load(reinterpret_cast<const HW_GLOBAL u32x4*>(addr + hh * 256));
                t.v[idx][hh * 4 + 0] = x.x;
                t.v[idx][hh * 4 + 1] = x.y;
                t.v[idx][hh * 4 + 2] = x.z;
                t.v[idx][hh * 4 + 3] = x.w;
            } else {
                const u32x2 x = __builtin_nontemporal_load(reinterpret_cast<const HW_GLOBAL u32x2*>(addr));
                t.v[idx][0] = x.x;
                t.v[idx][1] = x.y;
            }
        }
    }
}

// The wait in front of a tile's operand reads, stated by hand: the K transfers of the tile about to be multiplied have
// landed when at most the operations issued behind them are outstanding -- the tile's own V loads and everything of the
// AHEAD tiles requested after it (loads and transfers complete in issue order, and a tile is the same number of
// instructions whether or not it exists).  The compiler places this wait itself from its own count of the operations in
// flight, which ends at 63: with the 32 transfers + 32 loads of a 256-wide fp32 tile it placed none, and the operand reads
// raced with the transfers.  So the kernels state it wherever a tile and its look-ahead come to 64 operations or more
// (head dimension 256); where the compiler's own wait is present as well, the two agree.
template <class G, int AHEAD>
__device__ __forceinline__ void wait_k_landed() {
    constexpr int BEHIND = 8 * G::NVL + AHEAD * (G::KL + 8 * G::NVL);
    static_assert(BEHIND <= 63, "beyond the counter's range");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(BEHIND) : "memory");
}

// V image for transposed reads (the kernels whose waves share every tile, 16-bit types): rows of VROW bytes, the 32-byte
// segments of a row (16 elements: what one MFMA block of outputs needs) stored at segment ^ key(row), the key chosen so
// that the eight consecutive rows two neighbouring 16-lane groups read (2 x 4 rows x 32 bytes) cover all 64 banks:
// rows of 256 bytes start at bank 0, so the key is row & 7; rows of 128 bytes alternate between the two halves of the
// banks by themselves and the key is (row >> 1) & 3.
template <int VROW>
__device__ __forceinline__ int vimg_segment_key(int row) {
    static_assert(VROW == 256 || VROW == 128, "head dims 128 and 64 in 16-bit types");
    return VROW == 256 ? (row & 7) : ((row >> 1) & 3);
}

typedef short v4i16 __attribute__((ext_vector_type(4)));
// ds_read_b64_tr_b16: within a 16-lane group, lanes 4r .. 4r+3 name the four 8-byte pieces of row r (r = 0..3, 16
// elements), and lane d receives element d of rows 0..3: a 4 x 16 block delivered by columns, which is the MFMA operand
// layout of V^T (lane = output element, four consecutive tokens per read) without any register shuffling.
__device__ __forceinline__ u32x2 lds_read_tr16(const char* p) {
    const v4i16 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4i16*)(p));
    return __builtin_bit_cast(u32x2, r);
}
// Per-lane byte offsets into a swizzled V image for output block c (16 elements) and the first 16 tokens of a tile (the
// lane names row 4q + r, r = (lane / 4) % 4, piece lane % 4); add 16 * VROW for the second 16 tokens (same key).
template <int VROW>
__device__ __forceinline__ void vtr_lane_offsets(unsigned (&voff)[VROW / 32], int lane) {
    const int q = lane >> 4, r = (lane >> 2) & 3, j = lane & 3;
    const int row = q * 4 + r;
#pragma unroll
    for (int c = 0; c < VROW / 32; ++c) voff[c] = (unsigned)(row * VROW + ((c ^ vimg_segment_key<VROW>(row)) << 5) + 8 * j);
}

// Running state of one wave: RB row blocks of 16 rows each.
template <int RB, int NOC>
struct WaveState {
    f32x4 o[RB][NOC];
    float m[RB];   // reference of the exponentials (base-2 units): within 2^8 below/above the running max
    float l[RB];   // lane-partial sum: this lane's quarter of the tokens
    bool fresh;    // no tile accumulated yet (uniform over the wave)
};

// One 32-token tile against all rows.  MASKED = false is the fast path for tiles every row sees completely.
// VS = the logits S^T = K Q^T are formed with VALU dot products (v_dot2 / v_fma) instead of MFMA, in the same lane
// layout (row = lane % 16, eight tokens per lane): the measured alternative for workloads with few query rows.
// VLDS = the V rows of the tile lie in LDS as an image at `vimg`, swizzled for transposed reads (vimg_segment_key; the
// kernels whose waves share every tile, 16-bit types): the K operands are read first (LDS answers in order, and the
// logits wait for K only), the V^T operands come straight out of the image (lds_read_tr16, per-lane offsets `voff` from
// vtr_lane_offsets), and output block c then holds elements 16c .. 16c+15.  `t_in` is not used.
template <class DT, int E, int EV, int RB, bool MASKED, bool QREG, bool VS = false, bool VLDS = false>
__device__ __forceinline__ void compute_tile(const TileRegs<DT, E, EV>& t_in, const char* q_lds, const u32x4* qreg, const int (&lim)[RB],
                                             WaveState<RB, Geo<DT, E, EV>::NOC>& st, int t0, int n, int q, float sc, const char* kstage,
                                             const char* vimg = nullptr, const unsigned* voff = nullptr) {
    typedef Geo<DT, E, EV> G;
    const TileRegs<DT, E, EV>& t = t_in;
#ifdef HW_NO_COMPUTE   // tuning aid: consume the tile without doing the arithmetic
    {
        u32 x = 0;
#pragma unroll
        for (int idx = 0; idx < 8; ++idx)
#pragma unroll
            for (int d = 0; d < G::VW; ++d) x ^= t.v[idx][d];
        x ^= *reinterpret_cast<const u32*>(kstage + kstage_offset<G>(n, q));
        st.l[0] += __uint_as_float(x & 0x3fffffffu);
        return;
    }
#endif
    // K operand: out of the staging slot in MFMA A-operand order (lane = token, 16 B of head dim).  The compiler
    // tracks the outstanding global->LDS transfers per staging slot and waits for this slot's before the reads.
    // S^T blocks: for each 16-token block, its K operand (lane = token, 16 B of head dim per k-step) against the
    // B operand of every row block (this row's rotated query, from registers when QREG, else straight from LDS)
    f32x4 sacc[RB][2];
    if constexpr (VS) {
        // every lane walks the K rows of its own eight tokens (the 16 lanes of a quarter-wave read the same row: an
        // LDS broadcast) against its row's query, 16 bytes at a time
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
            for (int idx = 0; idx < 8; ++idx) {
                const int tok = slot_token(q, idx);
                float acc = 0.f;
#pragma unroll
                for (int c = 0; c < G::CPR; ++c) {
                    const u32x4 kk = *reinterpret_cast<const u32x4*>(kstage + kstage_offset<G>(tok, c));
                    const u32x4 qq = *reinterpret_cast<const u32x4*>(q_lds + (rb * 16 + n) * G::QSTR + c * 16);
#pragma unroll
                    for (int d = 0; d < 4; ++d) acc = Elem<DT>::dot(kk[d], qq[d], acc);
                }
                sacc[rb][idx >> 2][idx & 3] = acc;
            }
        }
    } else if constexpr (VLDS) {
        u32x4 kop[2][G::KJ];
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int j = 0; j < G::KJ; ++j) kop[tb][j] = *reinterpret_cast<const u32x4*>(kstage + kstage_offset<G>(tb * 16 + n, 4 * j + q));
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < G::KJ; ++j) acc = Elem<DT>::mfma(kop[tb][j], qreg[rb * G::KJ + j], acc);
                sacc[rb][tb] = acc;
            }
    } else
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
        u32x4 kop[G::KJ];
#pragma unroll
        for (int j = 0; j < G::KJ; ++j) kop[j] = *reinterpret_cast<const u32x4*>(kstage + kstage_offset<G>(tb * 16 + n, 4 * j + q));
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            u32x4 qop[G::KJ];
#pragma unroll
            for (int j = 0; j < G::KJ; ++j)
                qop[j] = QREG ? qreg[rb * G::KJ + j] : *reinterpret_cast<const u32x4*>(q_lds + (rb * 16 + n) * G::QSTR + (4 * j + q) * 16);
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            if constexpr (G::SZ == 2) {
#pragma unroll
                for (int j = 0; j < G::KJ; ++j) acc = Elem<DT>::mfma(kop[j], qop[j], acc);
            } else {
#pragma unroll
                for (int j = 0; j < G::KJ; ++j) {
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(kop[j][c]), __uint_as_float(qop[j][c]), acc, 0, 0, 0);
                }
            }
            sacc[rb][tb] = acc;
        }
    }
    // The V^T operands out of the LDS image, requested here: the LDS answers while the exponentials are taken, and the
    // output products below then issue back to back.  (Read where they are used, one chunk's pair of reads at a time into
    // the same registers, every chunk waited for the LDS round trip in front of its two products: eight exposed round
    // trips per tile.)
    [[maybe_unused]] u32x4 vops[VLDS ? G::NOC : 1];
    if constexpr (VLDS) {
#pragma unroll
        for (int c = 0; c < G::NOC; ++c) {
            const char* vp = vimg + voff[c];
            const u32x2 a0 = lds_read_tr16(vp), a1 = lds_read_tr16(vp + 16 * G::VROW);
            vops[c] = u32x4{a0.x, a0.y, a1.x, a1.y};     // tokens slot_token(q, 0..7) of element 16c + n
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    // Online softmax with a lazily updated reference: exponentials are taken against st.m, which only moves when
    // a row's maximum exceeds it by more than 2^LAZY_LOG2 (then O and l of that row are rescaled).  Most tiles
    // therefore leave the accumulators alone: no rescale multiplies, and O can stay in the MFMA accumulator
    // registers.  p is at most 2^LAZY_LOG2, far inside the range of every storage type.
    constexpr float LAZY_LOG2 = 8.0f;
    float s[RB][8];
    float mxl[RB];     // maximum over this lane's eight tokens (a quarter of the tile)
    bool need = false;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        float mx = NEG_BIG;
#pragma unroll
        for (int idx = 0; idx < 8; ++idx) {
            s[rb][idx] = sacc[rb][idx >> 2][idx & 3];
            if constexpr (MASKED) s[rb][idx] = (t0 + slot_token(q, idx)) < lim[rb] ? s[rb][idx] : NEG_BIG;
            mx = fmaxf(mx, s[rb][idx]);
        }
        mxl[rb] = mx;
        // A row's maximum exceeds the bound exactly when that of one of its four lanes does: the test needs no
        // reduction across the lanes, which is left to the (rare) branch that moves the reference.
        // sc > 0: scaling commutes with the max; a row that sees nothing of a masked tile keeps NEG_BIG
        const float mine = MASKED ? (mx < -1.0e29f ? NEG_BIG : mx * sc) : mx * sc;
        need = need || (mine > st.m[rb] + LAZY_LOG2);
    }
    if (__builtin_amdgcn_ballot_w64(need) != 0) {        // uniform over the wave
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const float mx = quarter_max(mxl[rb]);
            const float mxs = MASKED ? (mx < -1.0e29f ? NEG_BIG : mx * sc) : mx * sc;
            const float mnew = mxs > st.m[rb] + LAZY_LOG2 ? mxs : st.m[rb];
            const float alpha = fast_exp2(st.m[rb] - mnew);   // 1 for rows that keep their reference
            st.m[rb] = mnew;
            st.l[rb] *= alpha;
            if (!st.fresh) {                                  // before the first tile O is zero
#pragma unroll
                for (int c = 0; c < G::NOC; ++c) st.o[rb][c] *= alpha;
            }
        }
    }
    st.fresh = false;
    float p[RB][8];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        // a row that has seen nothing yet keeps the reference NEG_BIG; exponentiate against 0 so its masked slots give 0
        const float mref = MASKED ? (st.m[rb] < -1.0e29f ? 0.f : st.m[rb]) : st.m[rb];
        float psum;
#pragma unroll
        for (int idx = 0; idx < 8; ++idx) {
            p[rb][idx] = fast_exp2(__builtin_fmaf(s[rb][idx], sc, -mref));
            psum = idx == 0 ? p[rb][0] : psum + p[rb][idx];
        }
        st.l[rb] += psum;
    }

    if constexpr (G::SZ == 2) {
        u32x4 pp[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            pp[rb].x = Elem<DT>::pack2(p[rb][0], p[rb][1]);
            pp[rb].y = Elem<DT>::pack2(p[rb][2], p[rb][3]);
            pp[rb].z = Elem<DT>::pack2(p[rb][4], p[rb][5]);
            pp[rb].w = Elem<DT>::pack2(p[rb][6], p[rb][7]);
        }
        if constexpr (VLDS) {
#pragma unroll
            for (int c = 0; c < G::NOC; ++c) {
                const u32x4 vop = vops[c];
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) st.o[rb][c] = Elem<DT>::mfma(vop, pp[rb], st.o[rb][c]);
            }
        } else
        // dword d of a lane's V row holds two consecutive ev (out_ev(2d, n) and the next); gather the 8 tokens of each ev.
#pragma unroll
        for (int d = 0; d < G::VW; ++d) {
            u32x4 lo, hi;
            lo.x = __builtin_amdgcn_perm(t.v[1][d], t.v[0][d], 0x05040100u);
            lo.y = __builtin_amdgcn_perm(t.v[3][d], t.v[2][d], 0x05040100u);
            lo.z = __builtin_amdgcn_perm(t.v[5][d], t.v[4][d], 0x05040100u);
            lo.w = __builtin_amdgcn_perm(t.v[7][d], t.v[6][d], 0x05040100u);
            hi.x = __builtin_amdgcn_perm(t.v[1][d], t.v[0][d], 0x07060302u);
            hi.y = __builtin_amdgcn_perm(t.v[3][d], t.v[2][d], 0x07060302u);
            hi.z = __builtin_amdgcn_perm(t.v[5][d], t.v[4][d], 0x07060302u);
            hi.w = __builtin_amdgcn_perm(t.v[7][d], t.v[6][d], 0x07060302u);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                st.o[rb][2 * d] = Elem<DT>::mfma(lo, pp[rb], st.o[rb][2 * d]);
                st.o[rb][2 * d + 1] = Elem<DT>::mfma(hi, pp[rb], st.o[rb][2 * d + 1]);
            }
        }
    } else {
#pragma unroll
        for (int idx = 0; idx < 8; ++idx) {
#pragma unroll
            for (int c = 0; c < G::NOC; ++c) {
#pragma unroll
                for (int rb = 0; rb < RB; ++rb)
                    st.o[rb][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(t.v[idx][c]), p[rb][idx], st.o[rb][c], 0, 0, 0);
            }
        }
    }
}

// head-dim index of accumulator chunk c, accumulator row i (0..15)
template <class DT, int EV>
__device__ __forceinline__ int out_ev(int c, int i) {
    if constexpr (Elem<DT>::size == 2) {
        // lane i of a V row holds EV/16 consecutive elements -- of each 256-byte half, when the row has two (EV = 256)
        constexpr int CPL = EV / 16 > 8 ? 8 : EV / 16;
        return (c / CPL) * (16 * CPL) + i * CPL + (c % CPL);
    } else {
        return (c >> 2) * 64 + i * 4 + (c & 3);  // 16 lanes x 4 floats per 256-byte load, c>>2 selects the load
    }
}

// 16-byte chunk of CH elements <-> CH floats
template <class DT> struct Chunk;
template <> struct Chunk<F32> {
    static constexpr int CH = 4;
    static __device__ __forceinline__ void unpack(u32x4 x, float (&f)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(x[i]);
    }
    static __device__ __forceinline__ u32x4 pack(const float (&f)[4]) {
        return u32x4{__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
    }
};
template <> struct Chunk<BF16> {
    static constexpr int CH = 8;
    static __device__ __forceinline__ void unpack(u32x4 x, float (&f)[8]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(x[i] << 16);
            f[2 * i + 1] = __uint_as_float(x[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ u32x4 pack(const float (&f)[8]) {
        return u32x4{Elem<BF16>::pack2(f[0], f[1]), Elem<BF16>::pack2(f[2], f[3]), Elem<BF16>::pack2(f[4], f[5]),
                     Elem<BF16>::pack2(f[6], f[7])};
    }
};
template <> struct Chunk<F16> {
    static constexpr int CH = 8;
    static __device__ __forceinline__ void unpack(u32x4 x, float (&f)[8]) {
        f16x8 h = __builtin_bit_cast(f16x8, x);
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (float)h[i];
    }
    static __device__ __forceinline__ u32x4 pack(const float (&f)[8]) {
        return u32x4{Elem<F16>::pack2(f[0], f[1]), Elem<F16>::pack2(f[2], f[3]), Elem<F16>::pack2(f[4], f[5]),
                     Elem<F16>::pack2(f[6], f[7])};
    }
};


// What each wave of a workgroup hands over at the end: its accumulators exactly as the registers hold them (16 bytes
// per lane and accumulator, lane after lane: no bank conflicts, no register shuffling), and per row the four waves'
// references and sums next to each other (one 16-byte read fetches all of them).
template <int ROWS, int EV>
struct Exchange {
    static constexpr int NSLOT = (ROWS / 16) * (EV / 16);   // accumulators (f32x4 per lane) of one wave
    f32x4 o[NWAVES][NSLOT][64];
    float m[ROWS][NWAVES];
    float l[ROWS][NWAVES];
};

// Epilogue shared by the attention kernels: every wave hands over its raw accumulators, running max and sum
// through LDS (one barrier; the exchange is bound by LDS bandwidth: ~40 B/clk for one wave's writes, 128 B/clk for the
// workgroup's reads); then wave w combines accumulators w*NSLOT/4 ... of all four waves with the weights
// 2^(m_wave - m_max), still in the accumulator layout (row = lane % 16, so the weights are per-lane scalars), and
// stores its part of the workgroup's partial: `nrows` rows starting at partial row index `part` (EV floats per row
// in part_o, a (max, sum) pair per row in part_ml).  A wave's accumulators are consecutive 16-wide chunks of the head
// dimension whose elements interleave (out_ev), so a lane's values of SPW chunks form runs of SPW consecutive floats.
// The epilogue runs with one wave per SIMD, i.e. at the issue rate of a single wave: it is written for few
// instructions, not for few bytes.
// ALIASED: `ex` shares its memory with a K staging slot, so nobody may write it before every wave is done with its
// tiles; otherwise each wave hands over as soon as it is done, while the slower waves of the workgroup still compute.
// Rows beyond `nrows` (MFMA padding) are neither written nor read.
// `direct` (uniform over the launch): the workgroup holds everything its rows will ever see (one workgroup per kv head and
// row group), so the combined rows are normalised here and written as the operator's result: part_o is then the
// address of out, part_ml that of lse (or null), and orow[rb] the lane's output row (row index of out / lse) in row
// block rb.  The arithmetic is that of the merge kernel on a single partial, bit for bit.
template <class DT, int EV, int RB, bool ALIASED>
__device__ __forceinline__ void store_partials(WaveState<RB, EV / 16>& st, Exchange<RB * 16, EV>& ex, int wv, int n, int q, int tid,
                                               HW_GLOBAL float* part_o, HW_GLOBAL float* part_ml, size_t part, int nrows,
                                               bool direct = false, const size_t* orow = nullptr) {
    constexpr int NOC = EV / 16;
    constexpr int NSLOT = RB * NOC;
    constexpr int SPW = NSLOT / NWAVES;       // accumulators each wave combines
    static_assert(NWAVES == 4 && NSLOT % NWAVES == 0 && NOC % SPW == 0 && SPW <= 4, "a wave's share lies within one row block");
    const int lane = tid & 63;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) st.l[rb] = quarter_sum(st.l[rb]);
    if constexpr (ALIASED) {
        // a look-ahead transfer into the staging slot may still be in flight; it must have landed before ANY wave writes `ex`
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        const int row = rb * 16 + n;
        if (row < nrows) {
#pragma unroll
            for (int c = 0; c < NOC; ++c) ex.o[wv][rb * NOC + c][lane] = st.o[rb][c];
            if (q == 0) {
                ex.m[row][wv] = st.m[rb];
                ex.l[row][wv] = st.l[rb];
            }
        }
    }
    __syncthreads();
    HW_MARK(4);
    const int s0 = wv * SPW;                  // first accumulator of this wave's share
    const int rb = s0 / NOC, c0 = s0 % NOC;
    const int row = rb * 16 + n;
    if (row < nrows) {
        const f32x4 m4 = *reinterpret_cast<const f32x4*>(&ex.m[row][0]);
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(&ex.l[row][0]);
        f32x4 ov[SPW][NWAVES];
#pragma unroll
        for (int j = 0; j < SPW; ++j)
#pragma unroll
            for (int w2 = 0; w2 < NWAVES; ++w2) ov[j][w2] = ex.o[w2][s0 + j][lane];
        const float mm = fmaxf(fmaxf(m4[0], m4[1]), fmaxf(m4[2], m4[3]));
        float wgt[NWAVES];
#pragma unroll
        for (int w2 = 0; w2 < NWAVES; ++w2) wgt[w2] = fast_exp2(m4[w2] - mm);
        float lsum = 0.f;
#pragma unroll
        for (int w2 = 0; w2 < NWAVES; ++w2) lsum = __builtin_fmaf(l4[w2], wgt[w2], lsum);
        typedef typename Elem<DT>::store_t store_t;
        const size_t orw = direct ? orow[rb] : 0;
        const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
        HW_GLOBAL float* dst = part_o + (part + row) * EV;
        HW_GLOBAL store_t* odst = reinterpret_cast<HW_GLOBAL store_t*>(part_o) + orw * EV;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float run[SPW];
#pragma unroll
            for (int j = 0; j < SPW; ++j) {
                float acc = ov[j][0][i] * wgt[0];
#pragma unroll
                for (int w2 = 1; w2 < NWAVES; ++w2) acc = __builtin_fmaf(ov[j][w2][i], wgt[w2], acc);
                run[j] = acc;
            }
            const int e0 = out_ev<DT, EV>(c0, 4 * q + i);    // chunks c0 .. c0+SPW-1 are consecutive elements from here
            if (direct) {
#pragma unroll
                for (int j = 0; j < SPW; ++j) odst[e0 + j] = Elem<DT>::from_float(run[j] * inv);
            } else {
                HW_GLOBAL float* d = dst + e0;
                if constexpr (SPW == 4) *reinterpret_cast<HW_GLOBAL f32x4*>(d) = f32x4{run[0], run[1], run[2], run[3]};
                else if constexpr (SPW == 2) *reinterpret_cast<HW_GLOBAL f32x2*>(d) = f32x2{run[0], run[1]};
                else *d = run[0];
            }
        }
        if (q == 0 && c0 == 0) {
            if (!direct) *reinterpret_cast<HW_GLOBAL f32x2*>(part_ml + (part + row) * 2) = f32x2{mm, lsum};
            else if (part_ml != nullptr) part_ml[orw] = lsum > 0.f ? (mm + __builtin_amdgcn_logf(lsum)) * 0.69314718055994530942f : -__builtin_inff();
        }
    }
}


// KernelHeader as the kernel sees it after fetching it by hand: same layout, pointers typed as global memory
// (a pointer rebuilt from raw bits would otherwise be a flat pointer, and flat loads tie up both wait counters).
struct DevHeader {
    const HW_GLOBAL char* q;
    const HW_GLOBAL int* loc;
    const HW_GLOBAL float* cos;
    const HW_GLOBAL float* sin;
    HW_GLOBAL char* rq;
    HW_GLOBAL float* part_o;
    HW_GLOBAL float* part_ml;
    const HW_GLOBAL int* len_dev;
    int F, W, Hq, Hkv, S, R;
    int nrg, wgs_per_head, nwg;
    int slot_stride;
    int flags;
    float sc;
    unsigned magic_gq, magic_s, magic_nrg, magic_wg;
};
static_assert(sizeof(DevHeader) == sizeof(KernelHeader), "DevHeader mirrors KernelHeader");

// PagedHeader as the paged kernels see it after fetching it by hand (see DevHeader).
struct PagedDevHeader {
    const HW_GLOBAL char* q;
    const HW_GLOBAL int* loc;
    const HW_GLOBAL int* frag_len;
    const HW_GLOBAL char* kcache;
    const HW_GLOBAL char* vcache;
    const HW_GLOBAL int* block_table;
    const HW_GLOBAL int* cu_q;
    HW_GLOBAL float* part_o;
    HW_GLOBAL float* part_ml;
    int F, W, Hq, Hkv, LW, LS;
    int R;
    int block_size, max_blocks, num_blocks;
    int nsplit, nitems, nrg, nwg;
    int flags;
    float sc;
    unsigned magic_gq, magic_ls, magic_bs, magic_nsplit, magic_nitems, magic_nrg;
};
static_assert(sizeof(PagedDevHeader) == 160, "40 dwords of PagedHeader are fetched");
static_assert(offsetof(PagedHeader, pad) == 160, "PagedDevHeader mirrors the used part of PagedHeader");

// n / d for n < 2^20, d < 2^12 with the host-computed multiplier ceil(2^32 / d) mod 2^32: one multiply-high instead
// of the ~25-instruction integer division sequence.  d == 1 gives the multiplier 0, which stands for "n itself".
// Without a branch on purpose: the multiplier is uniform, a branch on it cuts the code around every division into basic
// blocks, and inside a tile loop the loads on either side then wait for each other instead of flying together.
__device__ __forceinline__ int fast_div(int n, unsigned magic) {
    const int by_one = magic == 0 ? -1 : 0;
    return (int)__umulhi((unsigned)n, magic) | (n & by_one);
}

// The 40 used dwords of a PagedHeader, fetched from the kernel-argument segment with three scalar loads: requested first
// thing in the kernel (the argument-independent setup runs while they are in flight), waited for and typed later.
typedef int hw_i32x16 __attribute__((ext_vector_type(16)));
typedef int hw_i32x8 __attribute__((ext_vector_type(8)));
struct PagedHeaderBits {
    hw_i32x16 lo, mid;
    hw_i32x8 hi;
};
__device__ __forceinline__ void paged_header_request(PagedHeaderBits& hb) {
    const auto argp = __builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("s_load_dwordx16 %0, %3, 0x0\n\ts_load_dwordx16 %1, %3, 0x40\n\ts_load_dwordx8 %2, %3, 0x80"
                 : "=&s"(hb.lo), "=&s"(hb.mid), "=&s"(hb.hi)
                 : "s"(argp)
                 : "memory");
}
__device__ __forceinline__ PagedDevHeader paged_header_wait(PagedHeaderBits& hb) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(hb.lo), "+s"(hb.mid), "+s"(hb.hi) : : "memory");
    struct RawHeader {
        int v[40];
    } raw;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        raw.v[i] = hb.lo[i];
        raw.v[16 + i] = hb.mid[i];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) raw.v[32 + i] = hb.hi[i];
    return __builtin_bit_cast(PagedDevHeader, raw);
}

// Work item of a paged launch -> (worker, row group of ROWS rows within the worker, query-token range of the worker).
// Fixed-length operator: nrg row groups per worker.  Packed queries (cu_q): row groups are numbered through the workers
// in order, and the worker whose range contains `item` is found with a wave-wide prefix sum over 64 workers at a time;
// found = false when the item lies beyond the last worker's row groups (the grid is sized for the worst case).
struct PagedItem {
    int w, rg, qs, qe;
    bool found;
};
template <int ROWS>
__device__ __forceinline__ PagedItem paged_item(const PagedDevHeader& ph, int item, int lane, int GQ) {
    PagedItem it = {0, 0, 0, 0, false};
    if (ph.cu_q == nullptr) {
        it.w = fast_div(item, ph.magic_nrg);
        it.rg = item - it.w * ph.nrg;
        it.qs = it.w * ph.LS;
        it.qe = it.qs + ph.LS;
        it.found = true;
    } else {
        int base = 0;
        for (int c = 0; c < ph.W && !it.found; c += 64) {
            const int idx = c + lane;
            const int a0 = ph.cu_q[min(idx, ph.W)], a1 = ph.cu_q[min(idx + 1, ph.W)];
            const int cnt = idx < ph.W ? (max(a1 - a0, 0) * GQ + ROWS - 1) / ROWS : 0;
            int inc = cnt;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) {
                const int v = __shfl_up(inc, off, 64);
                if (lane >= off) inc += v;
            }
            const int total = __builtin_amdgcn_readlane(inc, 63);
            if (item < base + total) {
                const int l0 = __builtin_ctzll(__ballot(base + inc > item));
                it.w = c + l0;
                it.rg = item - base - __builtin_amdgcn_readlane(inc - cnt, l0);
                it.qs = __builtin_amdgcn_readlane(a0, l0);
                it.qe = __builtin_amdgcn_readlane(a1, l0);
                it.found = true;
            }
            base += total;
        }
    }
    // a malformed prefix-sum array must not lead outside the buffers
    const int T = ph.LW * ph.LS;
    it.qe = min(it.qe, T);
    it.qs = min(max(it.qs, 0), it.qe);
    return it;
}


// row r (0..R) of a kv head -> (worker*S + token, q head, flat q row index)
struct RowMap {
    int ws;
    size_t qrow;
};
__device__ __forceinline__ RowMap map_row(const DevHeader& a, int r, int hkv, int GQ) {
    RowMap m;
    m.ws = fast_div(r, a.magic_gq);
    const int gq = r - m.ws * GQ;
    const int w = fast_div(m.ws, a.magic_s), s = m.ws - w * a.S;
    m.qrow = ((size_t)(w * a.Hq + hkv * GQ + gq) * a.S + s);
    return m;
}

// Query rotation of one fragment, split in two phases so that its few global loads can be issued BEFORE the
// K/V tile loads (loads return in issue order, so a dependent wait would otherwise drain the whole KV
// prefetch first) and consumed after them.  The kernel rotates over the full head dimension only (RotE == E,
// what the models on this path use); other rotary widths are rotated by the standalone kernel first and
// enter here as pre-rotated queries.  One work item = one 16-byte chunk pair (e, e + E/2) of one row; the
// item count per thread is a compile-time constant.  Index convention of src/rope.cuh:18-51: both halves
// read cos/sin at the first-half index.
// PRE = the queries arrive already rotated, [F,W,Hq,S,E] (the hogwild_sdpa entry): one item = one chunk copy.
template <class DT, int E, int ROWS, int QSTR, bool PRE, int NT = NTHREADS>
struct QueryRotation {
    static constexpr int SZ = Elem<DT>::size;
    static constexpr int CH = Chunk<DT>::CH;
    static constexpr int IPR = PRE ? E / CH : E / (2 * CH);                  // items per row
    static constexpr int NIT = (ROWS * IPR + NT - 1) / NT;       // items per thread

    u32x4 xa[NIT];
    u32x4 xb[PRE ? 1 : NIT];
    f32x4 cs[PRE ? 1 : NIT][CH / 4], sn[PRE ? 1 : NIT][CH / 4];

    __device__ __forceinline__ void load(const DevHeader& a, int f, int hkv, int r0, int GQ, int tid) {
        const size_t fstride = (size_t)a.W * a.Hq * a.S * E;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int item = tid + it * NT;
            const int rr = item / IPR, slot = item % IPR;
            // rows beyond R (MFMA padding) and threads beyond the item count read row 0: harmless, and keeps the
            // loads out of divergent control flow
            const int r = (item < ROWS * IPR && r0 + rr < a.R) ? r0 + rr : r0;
            const RowMap rm = map_row(a, r, hkv, GQ);
            const HW_GLOBAL char* qp = a.q + (rm.qrow * E + (PRE ? f * fstride : 0)) * SZ;
            xa[it] = *reinterpret_cast<const HW_GLOBAL u32x4*>(qp + slot * 16);
            if constexpr (!PRE) {
                xb[it] = *reinterpret_cast<const HW_GLOBAL u32x4*>(qp + (slot + IPR) * 16);
                const size_t co = ((size_t)f * a.W * a.S + rm.ws) * E + slot * CH;
#pragma unroll
                for (int i = 0; i < CH / 4; ++i) {
                    cs[it][i] = *reinterpret_cast<const HW_GLOBAL f32x4*>(a.cos + co + 4 * i);
                    sn[it][i] = *reinterpret_cast<const HW_GLOBAL f32x4*>(a.sin + co + 4 * i);
                }
            }
        }
    }

    __device__ __forceinline__ void finish(const DevHeader& a, char* q_lds, int f, int hkv, int r0, int GQ, bool write_rq,
                                           int tid) const {
        const size_t fstride = (size_t)a.W * a.Hq * a.S * E;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int item = tid + it * NT;
            const int rr = item / IPR, slot = item % IPR;
            if (item >= ROWS * IPR) continue;
            char* lrow = q_lds + rr * QSTR;
            const bool pad = r0 + rr >= a.R;   // padding rows of the 16-row MFMA block hold zeros
            const u32x4 z = {0, 0, 0, 0};
            if constexpr (PRE) {
                if (q_lds != nullptr) *reinterpret_cast<u32x4*>(lrow + slot * 16) = pad ? z : xa[it];
            } else {
                float x1[CH], x2[CH], y1[CH], y2[CH];
                Chunk<DT>::unpack(xa[it], x1);
                Chunk<DT>::unpack(xb[it], x2);
#pragma unroll
                for (int i = 0; i < CH; ++i) {
                    const float c = cs[it][i >> 2][i & 3], sv = sn[it][i >> 2][i & 3];
                    y1[i] = x1[i] * c - x2[i] * sv;
                    y2[i] = x2[i] * c + x1[i] * sv;
                }
                const u32x4 ya = Chunk<DT>::pack(y1), yb = Chunk<DT>::pack(y2);
                if (q_lds != nullptr) {     // (null: the rotated queries are only wanted in memory)
                    *reinterpret_cast<u32x4*>(lrow + slot * 16) = pad ? z : ya;
                    *reinterpret_cast<u32x4*>(lrow + (slot + IPR) * 16) = pad ? z : yb;
                }
                if (write_rq && !pad) {
                    const RowMap rm = map_row(a, r0 + rr, hkv, GQ);
                    HW_GLOBAL char* rqp = a.rq + (f * fstride + rm.qrow * E) * SZ;
                    *reinterpret_cast<HW_GLOBAL u32x4*>(rqp + slot * 16) = ya;
                    *reinterpret_cast<HW_GLOBAL u32x4*>(rqp + (slot + IPR) * 16) = yb;
                }
            }
        }
    }
};

// The same rotation done by every wave for itself, in the registers that hold the result as MFMA B operand: lane
// (n = lane % 16, q = lane / 16) holds, for each 16-row block rb, the 16-byte chunks 4j + q (j < KJ) of query row
// rb * 16 + n, and a rotation pair (e, e + E/2) is the chunk pair (4j + q, 4(j + KJ/2) + q): both in the same lane.  So
// a wave loads its own operands (and the cos/sin values of their first-half chunks, and its rows' locations) straight
// from memory, rotates them when they have arrived and starts on its tiles: no staging through LDS, no barrier, no
// waiting for the other waves of the workgroup.  The four waves load the same few KB (served by the L1).
template <class DT, int E, int RB, bool PRE>
struct LaneRotation {
    static constexpr int SZ = Elem<DT>::size;
    static constexpr int CH = Chunk<DT>::CH;
    static constexpr int KJ = E * SZ / 64;
    static constexpr int HJ = KJ / 2;
    static_assert(KJ % 2 == 0, "a rotation pair lies in one lane");

    u32x4 x[RB][KJ];
    f32x4 cs[PRE ? 1 : RB][PRE ? 1 : HJ][CH / 4], sn[PRE ? 1 : RB][PRE ? 1 : HJ][CH / 4];
    int lc[RB];

    __device__ __forceinline__ void load(const DevHeader& a, int f, int hkv, int r0, int GQ, int n, int q) {
        const size_t fstride = (size_t)a.W * a.Hq * a.S * E;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            // rows beyond R (MFMA padding) read the first row: harmless, and keeps the loads unconditional
            const int row = r0 + rb * 16 + n;
            const RowMap rm = map_row(a, row < a.R ? row : r0, hkv, GQ);
            const HW_GLOBAL char* qp = a.q + (rm.qrow * E + (PRE ? f * fstride : 0)) * SZ;
#pragma unroll
            for (int j = 0; j < KJ; ++j) x[rb][j] = *reinterpret_cast<const HW_GLOBAL u32x4*>(qp + (4 * j + q) * 16);
            if constexpr (!PRE) {
#pragma unroll
                for (int j = 0; j < HJ; ++j) {
                    const size_t co = ((size_t)f * a.W * a.S + rm.ws) * E + (4 * j + q) * CH;
#pragma unroll
                    for (int i = 0; i < CH / 4; ++i) {
                        cs[rb][j][i] = *reinterpret_cast<const HW_GLOBAL f32x4*>(a.cos + co + 4 * i);
                        sn[rb][j][i] = *reinterpret_cast<const HW_GLOBAL f32x4*>(a.sin + co + 4 * i);
                    }
                }
            }
            lc[rb] = a.loc[(size_t)f * a.W * a.S + rm.ws];
        }
    }

    // qreg[rb * KJ + j] = the operand of k-step j; lim[rb] = the row's visible length in this fragment of L tokens
    __device__ __forceinline__ void finish(const DevHeader& a, u32x4* qreg, int (&lim)[RB], int f, int hkv, int r0, int GQ, int L,
                                           bool write_rq, int n, int q) const {
        const size_t fstride = (size_t)a.W * a.Hq * a.S * E;
        const u32x4 z = {0, 0, 0, 0};
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const int row = r0 + rb * 16 + n;
            const bool pad = row >= a.R;          // padding rows of the 16-row MFMA block hold zeros and "see everything"
            lim[rb] = pad ? 0x7fffffff : min(L, max(0, lc[rb] + 1));
            if constexpr (PRE) {
#pragma unroll
                for (int j = 0; j < KJ; ++j) qreg[rb * KJ + j] = pad ? z : x[rb][j];
            } else {
                HW_GLOBAL char* rqp = nullptr;
                if (write_rq && !pad) rqp = a.rq + (f * fstride + map_row(a, row, hkv, GQ).qrow * E) * SZ;
#pragma unroll
                for (int j = 0; j < HJ; ++j) {
                    float x1[CH], x2[CH], y1[CH], y2[CH];
                    Chunk<DT>::unpack(x[rb][j], x1);
                    Chunk<DT>::unpack(x[rb][j + HJ], x2);
#pragma unroll
                    for (int i = 0; i < CH; ++i) {
                        const float c = cs[rb][j][i >> 2][i & 3], sv = sn[rb][j][i >> 2][i & 3];
                        y1[i] = x1[i] * c - x2[i] * sv;
                        y2[i] = x2[i] * c + x1[i] * sv;
                    }
                    const u32x4 ya = Chunk<DT>::pack(y1), yb = Chunk<DT>::pack(y2);
                    qreg[rb * KJ + j] = pad ? z : ya;
                    qreg[rb * KJ + j + HJ] = pad ? z : yb;
                    if (rqp != nullptr) {
                        *reinterpret_cast<HW_GLOBAL u32x4*>(rqp + (4 * j + q) * 16) = ya;
                        *reinterpret_cast<HW_GLOBAL u32x4*>(rqp + (4 * (j + HJ) + q) * 16) = yb;
                    }
                }
            }
        }
    }
};

}  // namespace hw
