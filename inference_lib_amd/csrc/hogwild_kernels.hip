// Hogwild! fragmented-KV decode attention for gfx950 (MI355X, CDNA4, wave64).
//
// One workgroup = one kv head x one contiguous range of 32-token tiles (crossing fragment boundaries)
// x up to 32 query rows, where a "row" is one (worker, token, q-head-in-group) triple.  All rows that
// share a kv head are multiplied against each K/V tile once, so KV is read from HBM once per step
// instead of once per (worker, token) as in the reference (src/kernels/kernel_v21.cuh:62-66).
//
// Per wave and tile:
//   S^T[token, row] = K[token, :] . Q[row, :]        v_mfma_f32_16x16x32 (bf16/f16) or 16x16x4 (f32)
//   online softmax in base 2 on the accumulator layout (rows live on lane%16, so every per-row scalar
//   is lane-local; only the row max needs two cross-lane steps)
//   O^T[ev, row] += V^T[ev, token] . P^T[token, row]
// K goes global -> VGPR straight into the A-operand layout (lane = token, 16 B of the head dim);
// V is loaded as whole 256-byte rows (16 lanes x 16 B) and transposed in registers with v_perm_b32,
// using the freedom to permute the reduced (token) index identically in both MFMA operands.
// The query is rotated per fragment in the prologue (src/rope.cuh:18-51), rounded to the storage type
// like the reference's `rq` scratch (src/rope.cuh:43-45) and kept in registers as the B operand.
//
// Partials (unnormalised O, running max, sum) go to the workspace; a second kernel merges them by
// log-sum-exp (the role of src/kernels/kernel_v21.cuh:605-656) and writes out + lse.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hogwild_kernels.h"

namespace hw {

// tile buffers per wave of the two-row-block 16-bit kernels (tuning knob)
#ifndef HW_PF2
#define HW_PF2 2
#endif
// waves per SIMD the two-row-block 16-bit kernels are register-budgeted for (tuning knob)
#ifndef HW_MINW2
#define HW_MINW2 1
#endif
#ifndef HW_VGPR_CAP
#define HW_VGPR_CAP
#endif

// Phase timestamps for kernel tuning; compiled in only with -DHW_CLOCKS (never in the shipped library).
#ifdef HW_CLOCKS
__device__ unsigned long long hw_clock_buf[4096 * 8];
#define HW_MARK(i)                                                                                  \
    do {                                                                                            \
        if ((threadIdx.x & 63) == 0 && blockIdx.x < 1024)                                           \
            hw_clock_buf[(blockIdx.x * 4 + (threadIdx.x >> 6)) * 8 + (i)] = wall_clock64();         \
    } while (0)
#else
#define HW_MARK(i) do { } while (0)
#endif

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
    static __device__ __forceinline__ f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};
template <> struct Elem<F32> {
    typedef float store_t;
    static constexpr int size = 4;
    static __device__ __forceinline__ float to_float(store_t x) { return x; }
    static __device__ __forceinline__ store_t from_float(float f) { return f; }
};

constexpr float NEG_BIG = -1.0e30f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// max over the four lanes {l, l^16, l^32, l^48}: the four quarter-waves hold different tokens of one row
__device__ __forceinline__ float quarter_max(float v) {
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}
__device__ __forceinline__ float quarter_sum(float v) {
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
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

// A fragment's K and V slices of one kv head as buffer resources: out-of-range rows read as zero, so tiles
// need no address clamping, and a tile that does not exist costs no memory traffic at all.
struct FragView {
    __amdgpu_buffer_rsrc_t k, v;
};
constexpr unsigned OOB_OFFSET = 0xFFFF0000u;   // beyond any fragment (lengths are validated on the host)

__device__ __forceinline__ FragView make_view(unsigned long long kptr, unsigned long long vptr, int hkv, int L, int krow, int vrow) {
    FragView fv;
    fv.k = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(kptr + (unsigned long long)hkv * L * krow), 0, L * krow, 0x00020000);
    fv.v = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(vptr + (unsigned long long)hkv * L * vrow), 0, L * vrow, 0x00020000);
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
// keeps the hardware wait counts exact on every path; a tile that does not exist reads out of range (zeros,
// no memory traffic).
template <class DT, int E, int EV>
__device__ __forceinline__ void load_tile(TileRegs<DT, E, EV>& t, const FragView& fv, char* kslot, const unsigned* koff, int t0,
                                          int n, int q, bool real) {
    typedef Geo<DT, E, EV> G;
    const unsigned kb = real ? (unsigned)(t0 * G::KROW) : OOB_OFFSET;
#pragma unroll
    for (int i = 0; i < G::KL; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(fv.k, HW_LDS_PTR(kslot + i * 1024), 16, kb + koff[i], 0, 0, 0);
    // V: a quarter-wave reads one whole row (or half of a 512-byte row) per load
    const unsigned vb = real ? (unsigned)((t0 + q * 4) * G::VROW + n * (G::VLD * 4)) : OOB_OFFSET;
#pragma unroll
    for (int idx = 0; idx < 8; ++idx) {
        const int rowoff = ((idx >> 2) * 16 + (idx & 3)) * G::VROW;
#pragma unroll
        for (int hh = 0; hh < G::NVL; ++hh) {
            if constexpr (G::VLD == 4) {
                const u32x4 x = __builtin_amdgcn_raw_buffer_load_b128(fv.v, vb + rowoff + hh * 256, 0, 0);
                t.v[idx][hh * 4 + 0] = x.x;
                t.v[idx][hh * 4 + 1] = x.y;
                t.v[idx][hh * 4 + 2] = x.z;
                t.v[idx][hh * 4 + 3] = x.w;
            } else {
                const u32x2 x = __builtin_amdgcn_raw_buffer_load_b64(fv.v, vb + rowoff, 0, 0);
                t.v[idx][0] = x.x;
                t.v[idx][1] = x.y;
            }
        }
    }
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
template <class DT, int E, int EV, int RB, bool MASKED, bool QREG>
__device__ __forceinline__ void compute_tile(const TileRegs<DT, E, EV>& t, const char* q_lds, const u32x4* qreg, const int (&lim)[RB],
                                             WaveState<RB, Geo<DT, E, EV>::NOC>& st, int t0, int n, int q, float sc, const char* kstage) {
    typedef Geo<DT, E, EV> G;
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
    // Online softmax with a lazily updated reference: exponentials are taken against st.m, which only moves when
    // a row's maximum exceeds it by more than 2^LAZY_LOG2 (then O and l of that row are rescaled).  Most tiles
    // therefore leave the accumulators alone: no rescale multiplies, and O can stay in the MFMA accumulator
    // registers.  p is at most 2^LAZY_LOG2, far inside the range of every storage type.
    constexpr float LAZY_LOG2 = 8.0f;
    float s[RB][8];
    float mxs[RB];
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
        mx = quarter_max(mx);
        mxs[rb] = mx < -1.0e29f ? NEG_BIG : mx * sc;      // sc > 0: scaling commutes with the max; nothing visible stays NEG_BIG
        need = need || (mxs[rb] > st.m[rb] + LAZY_LOG2);
    }
    if (__builtin_amdgcn_ballot_w64(need) != 0) {        // uniform over the wave
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const float mnew = mxs[rb] > st.m[rb] + LAZY_LOG2 ? mxs[rb] : st.m[rb];
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
        float psum = 0.f;
#pragma unroll
        for (int idx = 0; idx < 8; ++idx) {
            p[rb][idx] = fast_exp2(__builtin_fmaf(s[rb][idx], sc, -mref));
            psum += p[rb][idx];
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
        // dword d of a lane's V row holds ev (n*EVL + 2d, n*EVL + 2d + 1); gather the 8 tokens of each ev.
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
        return i * (EV / 16) + c;              // lane i of a V row holds EV/16 consecutive elements
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

#define HW_GLOBAL __attribute__((address_space(1)))

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
    int F, W, Hq, Hkv, S, RotE, R;
    int nrg, wgs_per_head, tiles_per_head, nwg;
    int prerotated;
    int xcd_remap;
    float sc;
    unsigned magic_gq, magic_s, magic_nrg, magic_wg;
};
static_assert(sizeof(DevHeader) == sizeof(KernelHeader), "DevHeader mirrors KernelHeader");

// n / d for n < 2^20, d < 2^12 with the host-computed multiplier ceil(2^32 / d) mod 2^32: one multiply-high instead
// of the ~25-instruction integer division sequence.  d == 1 gives the multiplier 0, which stands for "n itself".
__device__ __forceinline__ int fast_div(int n, unsigned magic) { return magic ? (int)__umulhi((unsigned)n, magic) : n; }

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
template <class DT, int E, int ROWS, int QSTR, bool PRE>
struct QueryRotation {
    static constexpr int SZ = Elem<DT>::size;
    static constexpr int CH = Chunk<DT>::CH;
    static constexpr int IPR = PRE ? E / CH : E / (2 * CH);                  // items per row
    static constexpr int NIT = (ROWS * IPR + NTHREADS - 1) / NTHREADS;       // items per thread

    u32x4 xa[NIT];
    u32x4 xb[PRE ? 1 : NIT];
    f32x4 cs[PRE ? 1 : NIT][CH / 4], sn[PRE ? 1 : NIT][CH / 4];

    __device__ __forceinline__ void load(const DevHeader& a, int f, int hkv, int r0, int GQ, int tid) {
        const size_t fstride = (size_t)a.W * a.Hq * a.S * E;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int item = tid + it * NTHREADS;
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
            const int item = tid + it * NTHREADS;
            const int rr = item / IPR, slot = item % IPR;
            if (item >= ROWS * IPR) continue;
            char* lrow = q_lds + rr * QSTR;
            const bool pad = r0 + rr >= a.R;   // padding rows of the 16-row MFMA block hold zeros
            const u32x4 z = {0, 0, 0, 0};
            if constexpr (PRE) {
                *reinterpret_cast<u32x4*>(lrow + slot * 16) = pad ? z : xa[it];
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
                *reinterpret_cast<u32x4*>(lrow + slot * 16) = pad ? z : ya;
                *reinterpret_cast<u32x4*>(lrow + (slot + IPR) * 16) = pad ? z : yb;
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

// MINW = waves per SIMD the register budget is sized for: 2 (<= 256 VGPRs) when one 16-row block is live,
// 1 (<= 512 VGPRs) when two row blocks or fp32 operands make the tile registers too large.
// PF = tiles a wave keeps in flight.  PRE = queries arrive rotated (hogwild_sdpa), else fused rotation.
template <class DT, int E, int EV, int RB, int MINW, int PF, bool PRE>
__global__ __launch_bounds__(NTHREADS, MINW) HW_VGPR_CAP void attention_kernel(const KernelArgs args) {
    typedef Geo<DT, E, EV> G;
    constexpr int ROWS = RB * 16;
    constexpr int SSTR = EV + 4;      // padded row stride of the epilogue exchange: rows land in different banks

    struct Exchange {                 // what each wave hands over at the end
        float o[NWAVES][ROWS][SSTR];
        float m[NWAVES][ROWS];
        float l[NWAVES][ROWS];
    };
    constexpr int SBYTES = NWAVES * G::KSTAGE;
    __shared__ __attribute__((aligned(16))) char q_lds[ROWS * G::QSTR];
    __shared__ int lim_lds[ROWS];
    // One K staging slot per tile in flight, each a separate LDS object so that the wait for a slot's incoming
    // transfers does not extend to the other slots.  The epilogue exchange reuses the memory of slot 0.
    union Slot0 {
        char k[SBYTES];
        Exchange ex;
    };
    __shared__ __attribute__((aligned(16))) Slot0 slot0;
    __shared__ __attribute__((aligned(16))) char slot1[PF > 1 ? SBYTES : 16];
    __shared__ __attribute__((aligned(16))) char slot2[PF > 2 ? SBYTES : 16];
    static_assert(PF <= 3, "three staging slots");

    const int tid = threadIdx.x;
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
    const int my_len = args.frag.len[fl];
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

    // consecutive logical ids stay on one XCD (hardware deals workgroups round-robin over the 8 XCDs)
    int bid = blockIdx.x;
    if (a.xcd_remap) bid = (bid & 7) * (a.nwg >> 3) + (bid >> 3);
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

    while (todo != 0) {
        const int f = __builtin_ctzll(todo);
        todo &= todo - 1;
        const int fb = __builtin_amdgcn_readlane(my_tb, f);
        const int fe = __builtin_amdgcn_readlane(my_te, f);
        const int s0 = max(T0, fb), s1 = min(T1, fe);
        const int L = __builtin_amdgcn_readlane(my_len, f);
        const unsigned long long kp = ((unsigned long long)(unsigned)__builtin_amdgcn_readlane((int)(my_k >> 32), f) << 32) |
                                      (unsigned)__builtin_amdgcn_readlane((int)my_k, f);
        const unsigned long long vp = ((unsigned long long)(unsigned)__builtin_amdgcn_readlane((int)(my_v >> 32), f) << 32) |
                                      (unsigned)__builtin_amdgcn_readlane((int)my_v, f);
        const FragView fv = make_view(kp, vp, hkv, L, G::KROW, G::VROW);
        const int lt0 = s0 - fb + wv;     // this wave's first tile of the segment (fragment-local)
        const int lt1 = s1 - fb;

        // global loads in issue order: query/cos/sin/loc of this fragment first (few), then the first PF
        // K/V tiles; the rotation then waits only for the former while the tiles stay in flight
        HW_MARK(6);
        QueryRotation<DT, E, ROWS, G::QSTR, PRE> qrot;
        qrot.load(a, f, hkv, r0, GQ, tid);
        HW_MARK(7);
        // (every thread loads, with a clamped row: a load inside a divergent branch would be waited for on the spot)
        const int lm = a.loc[(size_t)f * a.W * a.S + fast_div(min(r0 + (tid & (ROWS - 1)), a.R - 1), a.magic_gq)];
        // the first tile is requested before the prologue, further look-ahead tiles after it: a wave stalls
        // while the memory pipeline accepts its requests, and the prologue should not sit behind that stall
        TileRegs<DT, E, EV> tr[PF];
        if (PF > 1) load_tile<DT, E, EV>(tr[0], fv, kslots[0], koff, lt0 * TILE, n, q, lt0 < lt1);

        HW_MARK(1);
        // ---- prologue: rotate the queries of this fragment into LDS ----
        __syncthreads();   // previous segment's readers are done with q_lds / lim_lds
        qrot.finish(a, q_lds, f, hkv, r0, GQ, a.rq != nullptr && s0 == fb, tid);
        // rows that pad the MFMA block get "sees everything": their query is zero and they are never stored,
        // and they must not keep the unmasked fast path from being taken
        if (tid < ROWS) lim_lds[tid] = (r0 + tid < a.R) ? min(L, max(0, lm + 1)) : 0x7fffffff;
        __syncthreads();

        // with one wave per SIMD there are registers to spare: keep the query operands of the segment in them
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
            const bool pad = r0 + rb * 16 + n >= a.R;
            maxlim = max(maxlim, pad ? 0 : lim[rb]);
            minlim = min(minlim, lim[rb]);
        }
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
            maxlim = max(maxlim, __shfl_xor(maxlim, off, 64));
            minlim = min(minlim, __shfl_xor(minlim, off, 64));
        }
        maxlim = __builtin_amdgcn_readfirstlane(maxlim);
        minlim = __builtin_amdgcn_readfirstlane(minlim);
        HW_MARK(2);
#pragma unroll
        for (int i = 1; i < PF - 1; ++i)
            load_tile<DT, E, EV>(tr[i], fv, kslots[i], koff, (lt0 + i * NWAVES) * TILE, n, q, lt0 + i * NWAVES < lt1);

        // ---- stream this wave's tiles: PF buffers, the tile PF-1 steps ahead is requested right before each
        // tile is computed, so its transfer overlaps the arithmetic and the prologue above overlapped the first ----
        for (int lt = lt0; lt < lt1; lt += PF * NWAVES) {
#pragma unroll
            for (int i = 0; i < PF; ++i) {
                const int l = lt + i * NWAVES;
                const int t0 = l * TILE;
                const int nb = (i + PF - 1) % PF;   // constant after unrolling
                const int ln = l + (PF - 1) * NWAVES;
                load_tile<DT, E, EV>(tr[nb], fv, kslots[nb], koff, ln * TILE, n, q, ln < lt1);
                if (l < lt1 && t0 < maxlim) {
                    if (t0 + TILE <= minlim) compute_tile<DT, E, EV, RB, false, QREG>(tr[i], q_lds, qreg, lim, st, t0, n, q, a.sc, kslots[i]);
                    else compute_tile<DT, E, EV, RB, true, QREG>(tr[i], q_lds, qreg, lim, st, t0, n, q, a.sc, kslots[i]);
                }
            }
        }
    }

    HW_MARK(3);
    // ---- merge the four waves of the workgroup: every wave hands over its raw accumulators, running max and
    // sum; then all threads combine them with the weights 2^(m_wave - m_max) and store coalesced ----
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) st.l[rb] = quarter_sum(st.l[rb]);
    __syncthreads();   // every wave is done with K staging slot 0, whose memory the exchange buffer reuses
    Exchange& ex = slot0.ex;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
        for (int c = 0; c < G::NOC; ++c) {
#pragma unroll
            for (int i = 0; i < 4; ++i) ex.o[wv][rb * 16 + n][out_ev<DT, EV>(c, 4 * q + i)] = st.o[rb][c][i];
        }
        if (q == 0) {
            ex.m[wv][rb * 16 + n] = st.m[rb];
            ex.l[wv][rb * 16 + n] = st.l[rb];
        }
    }
    __syncthreads();
    HW_MARK(4);
    {
        const int nrows = min(ROWS, a.R - r0);
        const size_t part = (size_t)(hkv * a.wgs_per_head + g) * a.R + r0;
        HW_GLOBAL float* dst = a.part_o + part * EV;
        for (int idx = tid * 4; idx < nrows * EV; idx += NTHREADS * 4) {
            const int rr = idx / EV, e = idx - rr * EV;
            float mm = ex.m[0][rr];
#pragma unroll
            for (int w2 = 1; w2 < NWAVES; ++w2) mm = fmaxf(mm, ex.m[w2][rr]);
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            float lsum = 0.f;
#pragma unroll
            for (int w2 = 0; w2 < NWAVES; ++w2) {
                const float wgt = fast_exp2(ex.m[w2][rr] - mm);
                acc += *reinterpret_cast<const f32x4*>(&ex.o[w2][rr][e]) * wgt;
                lsum += ex.l[w2][rr] * wgt;
            }
            *reinterpret_cast<HW_GLOBAL f32x4*>(dst + idx) = acc;
            if (e == 0) {
                HW_GLOBAL float* ml = a.part_ml + (part + rr) * 2;
                ml[0] = mm;
                ml[1] = lsum;
            }
        }
    }
    HW_MARK(5);

    // rotated queries of zero-length fragments are still part of the operator's visible output
    if (!PRE && a.rq != nullptr && g == 0) {
        unsigned long long empty = __ballot(lane < a.F && my_len == 0);
        while (empty != 0) {
            const int f = __builtin_ctzll(empty);
            empty &= empty - 1;
            __syncthreads();
            QueryRotation<DT, E, ROWS, G::QSTR, PRE> qrot;
            qrot.load(a, f, hkv, r0, GQ, tid);
            qrot.finish(a, q_lds, f, hkv, r0, GQ, true, tid);
        }
    }
}

// Merge the split-K partials of one (kv head, row): out = sum_g 2^(m_g - M) O_g / sum_g 2^(m_g - M) l_g.
// Latency-bound, so everything a thread needs from global memory (its partial rows and their max/sum pairs) is
// requested in one batch before the first use; each thread then folds its partials with a running reference of
// its own, and the NPG partial groups are combined through LDS.
template <class DT, int EV>
__global__ __launch_bounds__(256) void merge_kernel(const MergeArgs a) {
    typedef typename Elem<DT>::store_t store_t;
    constexpr int V4 = EV / 4;          // threads along the head dim (4 floats each)
    constexpr int NPG = 256 / V4;       // partial groups
    constexpr int UN = 4;               // partials per thread and batch
    __shared__ __attribute__((aligned(16))) float red[NPG][EV];
    __shared__ float red_m[NPG], red_l[NPG];

    // Workgroups are dealt round-robin over the 8 XCDs.  When the attention kernel kept each kv head on one XCD, merge
    // that head's rows on the same XCD: its partials are then still in that XCD's L2.
    int hkv, r;
    if (a.xcd_local) {
        const int hpx = a.Hkv >> 3;                       // heads per XCD
        const int x = blockIdx.x & 7, j = blockIdx.x >> 3;
        hkv = x * hpx + j % hpx;
        r = j / hpx;
    } else {
        hkv = blockIdx.x / a.R;
        r = blockIdx.x - hkv * a.R;
    }
    const int tid = threadIdx.x;
    const int e4 = tid % V4, pg = tid / V4;
    const int ns = a.wgs_per_head;
    const float* ml = a.part_ml + ((size_t)hkv * ns * a.R + r) * 2;
    const size_t mstride = (size_t)a.R * 2;
    const float* po = a.part_o + ((size_t)hkv * ns * a.R + r) * EV + e4 * 4;
    const size_t ostride = (size_t)a.R * EV;

    float m_run = NEG_BIG, l_run = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = pg; s0 < ns; s0 += UN * NPG) {
        f32x4 o[UN];
        f32x2 mlv[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int s = s0 + u * NPG;
            const int sc = s < ns ? s : pg;                 // clamp: the loads stay unconditional
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
    if (pg == 0) {
        float M = red_m[0];
#pragma unroll
        for (int k = 1; k < NPG; ++k) M = fmaxf(M, red_m[k]);
        f32x4 tot = {0.f, 0.f, 0.f, 0.f};
        float L = 0.f;
#pragma unroll
        for (int k = 0; k < NPG; ++k) {
            const float w = fast_exp2(red_m[k] - M);
            tot += *reinterpret_cast<const f32x4*>(&red[k][e4 * 4]) * w;
            L += red_l[k] * w;
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

__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4* src, size_t n16, u32* sink) {
    u32x4 acc = {0, 0, 0, 0};
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) {
        u32x4 x = __builtin_nontemporal_load(src + i);
        acc ^= x;
    }
    u32 r = acc.x ^ acc.y ^ acc.z ^ acc.w;
    if (r == 0x9e3779b9u) sink[threadIdx.x] = r;   // practically never: keeps the loads alive without a store stream
}

__global__ __launch_bounds__(256) void stream_copy_kernel(u32x4* dst, const u32x4* src, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
template <class DT, int E, int EV, bool PRE>
static hipError_t launch_attention_rb(const KernelArgs& ka, int rb, hipStream_t stream) {
    constexpr bool half = Elem<DT>::size == 2;
    if (rb == 1)
        hipLaunchKernelGGL((attention_kernel<DT, E, EV, 1, half ? 2 : 1, half ? 2 : 1, PRE>), dim3(ka.h.nwg), dim3(NTHREADS), 0,
                           stream, ka);
    else
        hipLaunchKernelGGL((attention_kernel<DT, E, EV, 2, half ? HW_MINW2 : 1, half ? HW_PF2 : 1, PRE>), dim3(ka.h.nwg), dim3(NTHREADS), 0, stream, ka);
    return hipGetLastError();
}

template <class DT>
static hipError_t launch_attention_dt(const KernelArgs& ka, int E, int rb, hipStream_t stream) {
    if (ka.h.prerotated) {
        if (E == 128) return launch_attention_rb<DT, 128, 128, true>(ka, rb, stream);
        return launch_attention_rb<DT, 64, 64, true>(ka, rb, stream);
    }
    if (E == 128) return launch_attention_rb<DT, 128, 128, false>(ka, rb, stream);
    return launch_attention_rb<DT, 64, 64, false>(ka, rb, stream);
}

hipError_t launch_attention(const KernelArgs& ka, int dtype, int E, int rb, hipStream_t stream) {
    switch (dtype) {
        case 0: return launch_attention_dt<F32>(ka, E, rb, stream);
        case 1: return launch_attention_dt<F16>(ka, E, rb, stream);
        default: return launch_attention_dt<BF16>(ka, E, rb, stream);
    }
}

template <class DT>
static hipError_t launch_merge_dt(const MergeArgs& ma, int EV, hipStream_t stream) {
    const int blocks = ma.Hkv * ma.R;
    if (EV == 128)
        hipLaunchKernelGGL((merge_kernel<DT, 128>), dim3(blocks), dim3(256), 0, stream, ma);
    else
        hipLaunchKernelGGL((merge_kernel<DT, 64>), dim3(blocks), dim3(256), 0, stream, ma);
    return hipGetLastError();
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

hipError_t launch_stream_read(const void* src, size_t bytes, uint32_t* sink, hipStream_t stream) {
    hipLaunchKernelGGL(stream_read_kernel, dim3(2048), dim3(256), 0, stream, reinterpret_cast<const u32x4*>(src), bytes / 16, sink);
    return hipGetLastError();
}

hipError_t launch_stream_copy(void* dst, const void* src, size_t bytes, hipStream_t stream) {
    hipLaunchKernelGGL(stream_copy_kernel, dim3(2048), dim3(256), 0, stream, reinterpret_cast<u32x4*>(dst),
                       reinterpret_cast<const u32x4*>(src), bytes / 16);
    return hipGetLastError();
}

}  // namespace hw

#ifdef HW_CLOCKS
extern "C" int hw_debug_read_clocks(unsigned long long* host, size_t n) {
    return (int)hipMemcpyFromSymbol(host, HIP_SYMBOL(hw::hw_clock_buf), n * sizeof(unsigned long long));
}
#endif
