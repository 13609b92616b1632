// Caller-side steps around the Hogwild! attention path, for gfx950 (MI355X):
//
//   build_inputs_kernel ... locations / cosines / sines of a decode step for every (segment, worker, new token):
//                           what HogwildCache.update computes at layer 0 of the reference
//                           (python/hogwild/attention.py:164-196) with model.rotary_emb.
//   rope_append_kernel .... rotate the new keys (apply_rotary_pos_emb, python/hogwild/attention.py:84-90, called
//                           at :313-315) and append keys and values to each worker's segment
//                           (:148-158), in one pass and in place.  With one source "worker" and a single
//                           cos/sin row broadcast over its tokens this is also merge_caches (:251-257): re-rotate a
//                           whole segment by a constant offset and append it to another.
//   advance_lengths_kernel  len_dev[f] += add[f]: segment lengths kept in device memory, so that a decode step captured
//                           as a graph can be replayed while the segments grow (the first two kernels and the
//                           attention kernel then read the lengths from there).
//
// All are tiny, latency-bound kernels; they exist so that a decode step needs no per-worker Python loop, no
// torch.cat reallocation and no .contiguous() copy of the segments.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hogwild_kernels.h"
#include "hogwild_device.h"

namespace hw {

template <int ROUND>   // 0 = keep fp32, 1 = round to fp16, 2 = round to bf16 (values stay stored as fp32)
__device__ __forceinline__ float round_table(float x) {
    if constexpr (ROUND == 1) return (float)(_Float16)x;
    if constexpr (ROUND == 2) return (float)(__bf16)x;
    return x;
}

template <int ROUND>
__global__ __launch_bounds__(256) void build_inputs_kernel(const BuildInputsArgs a) {
    const int half = a.RotE >> 1;
    const int per_tok = half > 0 ? half : 1;
    const int total = a.F * a.W * a.S * per_tok;
    for (int idx = blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += gridDim.x * blockDim.x) {
        const int i = idx % per_tok;
        const int tok = idx / per_tok;            // (f * W + w) * S + s
        const int s = tok % a.S;
        const int fw = tok / a.S;
        int pos_end;
        if (a.len_dev == nullptr) {
            pos_end = a.pos_end[fw];
        } else {   // lengths in device memory: walk worker w's order from its end up to fragment f
            const int f = fw / a.W, w = fw - f * a.W;
            pos_end = 0;
            for (int i = a.F - 1; i >= 0; --i) {
                const int g = a.pos_end[w * a.F + i];
                pos_end += a.len_dev[g];
                if (g == f) break;
            }
        }
        const int pos = pos_end - a.S + s;
        if (i == 0) a.locations[tok] = pos;
        if (half > 0) {
            // angle = float(position) * inv_freq, then cos / sin times the attention scaling, as the rotary
            // embedding modules of the model library compute them in fp32
            const float ang = (float)pos * a.inv_freq[i];
            const float c = round_table<ROUND>(cosf(ang) * a.scaling);
            const float sn = round_table<ROUND>(sinf(ang) * a.scaling);
            float* cr = a.cosines + (size_t)tok * a.RotE;
            float* sr = a.sines + (size_t)tok * a.RotE;
            cr[i] = c;
            cr[i + half] = c;
            sr[i] = sn;
            sr[i + half] = sn;
        }
    }
}

// Rounds an fp32 intermediate to the type an eager tensor expression would hold it in.
template <class DT>
__device__ __forceinline__ float to_storage(float x) {
    return Elem<DT>::to_float(Elem<DT>::from_float(x));
}

// One (first-half, second-half) element pair of a rotated key.  EAGER reproduces the evaluation order and the
// roundings of `(x * cos) + (rotate_half(x) * sin)` on tensors: every product and the sum are rounded to the common
// type of x and cos/sin (16-bit tables: the 16-bit type; fp32 tables: fp32), the result to the type of x.
template <class DT, bool EAGER, bool CS16>
__device__ __forceinline__ void rotate_pair(float x1, float x2, float c1, float s1, float c2, float s2, float& y1, float& y2) {
    if constexpr (EAGER) {
#pragma clang fp contract(off)
        float a1 = x1 * c1, b1 = x2 * s1, a2 = x2 * c2, b2 = x1 * s2;
        if constexpr (CS16) {
            a1 = to_storage<DT>(a1);
            b1 = to_storage<DT>(b1);
            a2 = to_storage<DT>(a2);
            b2 = to_storage<DT>(b2);
        }
        y1 = a1 - b1;
        y2 = a2 + b2;
    } else {
        y1 = x1 * c1 - x2 * s1;
        y2 = x2 * c2 + x1 * s2;
    }
}

template <class DT, bool CS16>
__device__ __forceinline__ float load_cs(const void* base, long long idx) {
    if constexpr (CS16) return Elem<DT>::to_float(reinterpret_cast<const typename Elem<DT>::store_t*>(base)[idx]);
    else return reinterpret_cast<const float*>(base)[idx];
}

// grid = (blocks over the items of one worker, worker).  VEC = 16-byte chunks (head dims, rotary half-width and all
// strides multiples of a chunk) or single elements.
template <class DT, bool EAGER, bool CS16, bool VEC>
__global__ __launch_bounds__(256) void rope_append_kernel(const AppendArgs a) {
    typedef typename Elem<DT>::store_t store_t;
    constexpr int SZ = Elem<DT>::size;
    constexpr int CH = VEC ? Chunk<DT>::CH : 1;
    const int w = blockIdx.y;
    const int n_new = a.n_new[w];
    if (n_new <= 0) return;
    const int half = a.RotE >> 1;
    const int n_pair = half / CH, n_pass = (a.E - a.RotE) / CH, n_v = a.Ev / CH;
    const int per_row = n_pair + n_pass + n_v;
    const long long total = (long long)n_new * a.Hkv * per_row;
    const int s_first = a.S - n_new;                 // left masking: the last n_new tokens are the real ones
    const char* ksrc = reinterpret_cast<const char*>(a.k_src);
    const char* vsrc = reinterpret_cast<const char*>(a.v_src);
    char* kdst = reinterpret_cast<char*>(a.k_dst[w]);
    char* vdst = reinterpret_cast<char*>(a.v_dst[w]);
    const int cap = a.dst_cap[w];
    // rows already in the segment: given, or (lengths in device memory) the segment's length after this append minus
    // what is being appended; an append that would not fit is dropped rather than written outside the buffers
    const int len = a.len_dev == nullptr ? a.dst_len[w] : a.len_dev[a.dst_len[w]] - n_new;
    if (len < 0 || len + n_new > cap) return;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long long)gridDim.x * blockDim.x) {
        const int c = (int)(idx % per_row);
        const long long row = idx / per_row;
        const int t = (int)(row % n_new);
        const int h = (int)(row / n_new);
        const int s = s_first + t;
        const size_t drow = (size_t)h * cap + len + t;
        if (c < n_pair) {
            const char* src = ksrc + ((long long)w * a.ks_w + (long long)h * a.ks_h + (long long)s * a.ks_s) * SZ;
            char* dst = kdst + drow * a.E * SZ;
            const long long cs = (long long)w * a.cs_w + (long long)s * a.cs_s;
            const int e1 = c * CH, e2 = e1 + half;
            if constexpr (VEC) {
                float x1[CH], x2[CH], y1[CH], y2[CH];
                Chunk<DT>::unpack(*reinterpret_cast<const u32x4*>(src + e1 * SZ), x1);
                Chunk<DT>::unpack(*reinterpret_cast<const u32x4*>(src + e2 * SZ), x2);
#pragma unroll
                for (int i = 0; i < CH; ++i) {
                    const float c1 = load_cs<DT, CS16>(a.cos, cs + e1 + i), s1 = load_cs<DT, CS16>(a.sin, cs + e1 + i);
                    const float c2 = load_cs<DT, CS16>(a.cos, cs + e2 + i), s2 = load_cs<DT, CS16>(a.sin, cs + e2 + i);
                    rotate_pair<DT, EAGER, CS16>(x1[i], x2[i], c1, s1, c2, s2, y1[i], y2[i]);
                }
                *reinterpret_cast<u32x4*>(dst + e1 * SZ) = Chunk<DT>::pack(y1);
                *reinterpret_cast<u32x4*>(dst + e2 * SZ) = Chunk<DT>::pack(y2);
            } else {
                const store_t* sp = reinterpret_cast<const store_t*>(src);
                store_t* dp = reinterpret_cast<store_t*>(dst);
                float y1, y2;
                rotate_pair<DT, EAGER, CS16>(Elem<DT>::to_float(sp[e1]), Elem<DT>::to_float(sp[e2]), load_cs<DT, CS16>(a.cos, cs + e1),
                                             load_cs<DT, CS16>(a.sin, cs + e1), load_cs<DT, CS16>(a.cos, cs + e2),
                                             load_cs<DT, CS16>(a.sin, cs + e2), y1, y2);
                dp[e1] = Elem<DT>::from_float(y1);
                dp[e2] = Elem<DT>::from_float(y2);
            }
        } else if (c < n_pair + n_pass) {
            const int e = a.RotE + (c - n_pair) * CH;
            const char* src = ksrc + ((long long)w * a.ks_w + (long long)h * a.ks_h + (long long)s * a.ks_s) * SZ + e * SZ;
            char* dst = kdst + drow * a.E * SZ + e * SZ;
            if constexpr (VEC) *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(src);
            else *reinterpret_cast<store_t*>(dst) = *reinterpret_cast<const store_t*>(src);
        } else {
            const int e = (c - n_pair - n_pass) * CH;
            const char* src = vsrc + ((long long)w * a.vs_w + (long long)h * a.vs_h + (long long)s * a.vs_s) * SZ + e * SZ;
            char* dst = vdst + drow * a.Ev * SZ + e * SZ;
            if constexpr (VEC) *reinterpret_cast<u32x4*>(dst) = *reinterpret_cast<const u32x4*>(src);
            else *reinterpret_cast<store_t*>(dst) = *reinterpret_cast<const store_t*>(src);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// launchers
// ------------------------------------------------------------------------------------------------
hipError_t launch_build_inputs(const BuildInputsArgs& a, int round_dtype, hipStream_t stream) {
    const long long total = (long long)a.F * a.W * a.S * ((a.RotE >> 1) > 0 ? (a.RotE >> 1) : 1);
    if (total <= 0) return hipSuccess;
    long long blocks = (total + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    switch (round_dtype) {
        case 1: hipLaunchKernelGGL((build_inputs_kernel<1>), dim3((unsigned)blocks), dim3(256), 0, stream, a); break;
        case 2: hipLaunchKernelGGL((build_inputs_kernel<2>), dim3((unsigned)blocks), dim3(256), 0, stream, a); break;
        default: hipLaunchKernelGGL((build_inputs_kernel<0>), dim3((unsigned)blocks), dim3(256), 0, stream, a); break;
    }
    return hipGetLastError();
}

__global__ __launch_bounds__(64) void advance_lengths_kernel(const AdvanceArgs a) {
    const int f = threadIdx.x;
    if (f < a.F) a.len_dev[f] += a.add[f];
}

hipError_t launch_advance_lengths(const AdvanceArgs& a, hipStream_t stream) {
    hipLaunchKernelGGL(advance_lengths_kernel, dim3(1), dim3(64), 0, stream, a);
    return hipGetLastError();
}

template <class DT, bool EAGER, bool CS16>
static hipError_t launch_append_v(const AppendArgs& a, bool vec, dim3 grid, hipStream_t stream) {
    if (vec) hipLaunchKernelGGL((rope_append_kernel<DT, EAGER, CS16, true>), grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((rope_append_kernel<DT, EAGER, CS16, false>), grid, dim3(256), 0, stream, a);
    return hipGetLastError();
}

template <class DT>
static hipError_t launch_append_dt(const AppendArgs& a, bool eager, bool cs16, bool vec, dim3 grid, hipStream_t stream) {
    if constexpr (Elem<DT>::size == 2) {
        if (cs16) return eager ? launch_append_v<DT, true, true>(a, vec, grid, stream) : launch_append_v<DT, false, true>(a, vec, grid, stream);
    }
    return eager ? launch_append_v<DT, true, false>(a, vec, grid, stream) : launch_append_v<DT, false, false>(a, vec, grid, stream);
}

hipError_t launch_rope_append(const AppendArgs& a, int dtype, bool eager, bool cs16, hipStream_t stream) {
    const int sz = dtype == 0 ? 4 : 2;
    const int ch = 16 / sz;
    int max_new = 0;
    bool aligned = true;
    for (int w = 0; w < a.W; ++w) {
        if (a.n_new[w] > max_new) max_new = a.n_new[w];
        aligned = aligned && ((reinterpret_cast<uintptr_t>(a.k_dst[w]) | reinterpret_cast<uintptr_t>(a.v_dst[w])) & 15u) == 0;
    }
    if (max_new <= 0) return hipSuccess;
    const int half = a.RotE >> 1;
    auto mult = [&](long long v) { return (v * sz) % 16 == 0; };
    const bool vec = aligned && a.E % ch == 0 && a.Ev % ch == 0 && half % ch == 0 && mult(a.ks_w) && mult(a.ks_h) && mult(a.ks_s) &&
                     mult(a.vs_w) && mult(a.vs_h) && mult(a.vs_s) &&
                     ((reinterpret_cast<uintptr_t>(a.k_src) | reinterpret_cast<uintptr_t>(a.v_src)) & 15u) == 0;
    const int c = vec ? ch : 1;
    const long long per_row = half / c + (a.E - a.RotE) / c + a.Ev / c;
    long long blocks = ((long long)max_new * a.Hkv * per_row + 255) / 256;
    if (blocks > 2048) blocks = 2048;
    if (blocks < 1) blocks = 1;
    const dim3 grid((unsigned)blocks, (unsigned)a.W);
    switch (dtype) {
        case 0: return launch_append_dt<F32>(a, eager, false, vec, grid, stream);
        case 1: return launch_append_dt<F16>(a, eager, cs16, vec, grid, stream);
        default: return launch_append_dt<BF16>(a, eager, cs16, vec, grid, stream);
    }
}

}  // namespace hw
