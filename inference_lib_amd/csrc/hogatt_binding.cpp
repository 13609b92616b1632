// PyTorch operator binding for the MI355X Hogwild! attention library.
//
// Registers the operators of the reference's namespace `libhogatt` (the fused decode path and its paged
// variants), with the same schema strings (src/binding.cu:363-374 of the reference), on the dispatch key ROCm tensors use
// (CUDA).  Every operator only unpacks tensors into the plain-pointer hw_problem of include/hogwild_hip.h and
// calls the C ABI on the current HIP stream; no device code lives here.
//
// Differences from the reference binding, all deliberate:
//   * work is queued on the caller's current stream (the reference launches on the default stream,
//     src/rope.cuh:61, src/kernels/kernel_v21.cuh:985,989);
//   * an unsupported dtype or head dimension raises instead of silently doing nothing
//     (src/binding.cu:260-266, src/kernels/kernel_v21.cuh:992-995);
//   * the split-K workspace comes from the caching allocator per call instead of a leaked static
//     (src/kernels/kernel_v21.cuh:969-980), and the fragment pointers travel in the kernel arguments instead
//     of a host-to-device copy per call (src/binding.cu:77-103);
//   * `fragment_lengths` is accepted for schema compatibility; the lengths are read from the fragment sizes,
//     which the reference requires to be equal to it (src/kernels/kernel_v21.cuh:116-117);
//   * `hogwild_fused_lse` / `hogwild_sdpa_lse` additionally return the log-sum-exp per query row;
//   * `hogwild_fused_devlen` takes the current fragment lengths from `fragment_lengths` in device memory.

#include <ATen/Tensor.h>
#include <ATen/ops/empty.h>
#include <Python.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <string>
#include <vector>

#include "hogwild_hip.h"

namespace {

int dtype_code(const at::Tensor& t) {
    switch (t.scalar_type()) {
        case at::kFloat: return HW_F32;
        case at::kHalf: return HW_F16;
        case at::kBFloat16: return HW_BF16;
        default: TORCH_CHECK(false, "libhogatt: unsupported dtype ", t.scalar_type(), " (need float32, float16 or bfloat16)");
    }
}

void check_status(int status, const char* where) {
    TORCH_CHECK(status == 0, "libhogatt::", where, " failed with status ", status, ": ", hw_status_string(status));
}

// Drops the optional leading batch dimension of 1 of a KV fragment: [1, Hkv, L, D] -> [Hkv, L, D].
at::Tensor fragment_view(const at::Tensor& t, const char* what, size_t f) {
    TORCH_CHECK(t.dim() == 3 || (t.dim() == 4 && t.size(0) == 1), "libhogatt: ", what, " fragment ", f,
                " must be [Hkv, L, D] or [1, Hkv, L, D], got ", t.sizes());
    return t.dim() == 4 ? t.select(0, 0) : t;
}

// Rows between consecutive kv heads of a fragment [Hkv, L, D] whose rows are contiguous, or -1 if the pair of tensors is
// not of that form (packed fragments give L).
int64_t row_capacity(const at::Tensor& k, const at::Tensor& v) {
    const int64_t Hkv = k.size(0), L = k.size(1), E = k.size(2), Ev = v.size(2);
    if (L == 0) return 0;
    if ((E > 1 && k.stride(2) != 1) || (Ev > 1 && v.stride(2) != 1)) return -1;
    if (L > 1 && (k.stride(1) != E || v.stride(1) != Ev)) return -1;
    if (Hkv == 1) return L;
    if (k.stride(0) % E != 0 || v.stride(0) % Ev != 0 || k.stride(0) / E != v.stride(0) / Ev || k.stride(0) / E < L) return -1;
    return k.stride(0) / E;
}

struct Unpacked {
    hw_problem p{};
    std::vector<at::Tensor> keep;          // contiguous fragment tensors kept alive until the launch is queued
    std::vector<const void*> kptr, vptr;
    std::vector<int32_t> len, cap;
    at::Tensor workspace;
};

// Shape checks shared by the fused and the pre-rotated entry (the checks of src/binding.cu:47-97, as errors).
void unpack_common(Unpacked& u, at::Tensor& out, double scale, const at::Tensor& locations, const at::Tensor& queries,
                   const at::Tensor& fragment_lengths, const std::vector<at::Tensor>& key_fragments,
                   const std::vector<at::Tensor>& value_fragments, bool prerotated, bool copy_noncontiguous) {
    TORCH_CHECK(out.dim() == 4, "libhogatt: output must be [W, Hq, S, Ev]");
    TORCH_CHECK(out.is_contiguous(), "libhogatt: output must be contiguous");
    const int64_t W = out.size(0), Hq = out.size(1), S = out.size(2), Ev = out.size(3);
    const int64_t F = locations.size(0);
    TORCH_CHECK(locations.dim() == 3 && locations.size(1) == W && locations.size(2) == S, "libhogatt: locations must be [F, W, S]");
    TORCH_CHECK(locations.scalar_type() == at::kInt && locations.is_contiguous(), "libhogatt: locations must be contiguous int32");
    TORCH_CHECK((int64_t)key_fragments.size() == F && (int64_t)value_fragments.size() == F,
                "libhogatt: need one key and one value fragment per row of locations");
    TORCH_CHECK(F >= 1 && F <= HW_MAX_FRAGMENTS, "libhogatt: fragment count ", F, " outside 1..", HW_MAX_FRAGMENTS);
    TORCH_CHECK(fragment_lengths.dim() == 1 && fragment_lengths.size(0) == F, "libhogatt: fragment_lengths must be [F]");
    TORCH_CHECK(queries.is_contiguous(), "libhogatt: queries must be contiguous");
    TORCH_CHECK(queries.scalar_type() == out.scalar_type(), "libhogatt: queries and output must have the same dtype");
    const int64_t E = queries.size(-1);
    if (prerotated) {
        TORCH_CHECK(queries.dim() == 5 && queries.size(0) == F && queries.size(1) == W && queries.size(2) == Hq && queries.size(3) == S,
                    "libhogatt: rotated queries must be [F, W, Hq, S, E]");
    } else {
        TORCH_CHECK(queries.dim() == 4 && queries.size(0) == W && queries.size(1) == Hq && queries.size(2) == S,
                    "libhogatt: queries must be [W, Hq, S, E]");
    }
    u.kptr.resize(F);
    u.vptr.resize(F);
    u.len.resize(F);
    u.cap.resize(F);
    int64_t Hkv = -1;
    for (int64_t f = 0; f < F; ++f) {
        at::Tensor k = fragment_view(key_fragments[f], "key", f);
        at::Tensor v = fragment_view(value_fragments[f], "value", f);
        if (f == 0) Hkv = k.size(0);
        TORCH_CHECK(k.size(0) == Hkv && v.size(0) == Hkv, "libhogatt: fragment ", f, " has a different number of kv heads");
        TORCH_CHECK(k.size(1) == v.size(1), "libhogatt: key and value fragment ", f, " differ in length");
        TORCH_CHECK(k.size(2) == E && v.size(2) == Ev, "libhogatt: fragment ", f, " has the wrong head dimension");
        TORCH_CHECK(k.scalar_type() == out.scalar_type() && v.scalar_type() == out.scalar_type(),
                    "libhogatt: fragment ", f, " has a different dtype than the output");
        TORCH_CHECK(k.device() == out.device() && v.device() == out.device(), "libhogatt: fragment ", f, " lives on another device");
        // A fragment may be a view into a [Hkv, cap, D] allocation that grows in place: rows contiguous, kv heads a
        // whole number of rows apart.  Anything else is copied by the fused op (as the reference does,
        // src/binding.cu:330-337) and rejected by hogwild_sdpa.
        int64_t cap = row_capacity(k, v);
        if (cap < 0 && copy_noncontiguous) {
            k = k.contiguous();
            v = v.contiguous();
            cap = k.size(1);
        }
        TORCH_CHECK(cap >= 0, "libhogatt: fragment ", f, " must be contiguous (or have contiguous rows and kv heads a whole "
                    "number of rows apart, the same for keys and values)");
        u.kptr[f] = k.const_data_ptr();
        u.vptr[f] = v.const_data_ptr();
        u.len[f] = (int32_t)k.size(1);
        u.cap[f] = (int32_t)cap;
        u.keep.push_back(k);
        u.keep.push_back(v);
    }
    TORCH_CHECK(Hkv > 0 && Hq % Hkv == 0, "libhogatt: Hq must be a multiple of Hkv");
    hw_problem& p = u.p;
    p.dtype = dtype_code(out);
    p.F = (int32_t)F;
    p.W = (int32_t)W;
    p.Hq = (int32_t)Hq;
    p.Hkv = (int32_t)Hkv;
    p.S = (int32_t)S;
    p.E = (int32_t)E;
    p.Ev = (int32_t)Ev;
    p.scale = (float)scale;
    p.out = out.data_ptr();
    p.q = queries.const_data_ptr();
    p.locations = locations.const_data_ptr<int32_t>();
    p.k = u.kptr.data();
    p.v = u.vptr.data();
    p.len = u.len.data();
    p.cap = u.cap.data();
}

void run(Unpacked& u, const at::Tensor& out, bool fused) {
    c10::hip::HIPGuardMasqueradingAsCUDA guard(out.device());   // ROCm tensors report the device type "cuda"
    size_t bytes = 0;
    if (fused)
        check_status(hw_workspace_bytes(&u.p, &bytes), "hw_workspace_bytes");
    else
        check_status(hw_sdpa_workspace_bytes(&u.p, &bytes), "hw_sdpa_workspace_bytes");
    u.workspace = at::empty({(int64_t)bytes}, out.options().dtype(at::kByte));
    u.p.workspace = u.workspace.data_ptr();
    u.p.workspace_bytes = bytes;
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(out.device().index()).stream();
    if (fused)
        check_status(hw_fused_attention(&u.p, stream), "hw_fused_attention");
    else
        check_status(hw_sdpa(&u.p, stream), "hw_sdpa");
}

void attach_lse(Unpacked& u, const at::Tensor& out, at::Tensor& lse) {
    TORCH_CHECK(lse.scalar_type() == at::kFloat && lse.is_contiguous() && lse.dim() == 3 && lse.size(0) == out.size(0) &&
                    lse.size(1) == out.size(1) && lse.size(2) == out.size(2),
                "libhogatt: lse must be contiguous float32 [W, Hq, S]");
    u.p.lse = lse.data_ptr<float>();
}

void attach_rotation(Unpacked& u, const at::Tensor& out, at::Tensor& rq, const at::Tensor& cosines, const at::Tensor& sines) {
    const hw_problem& p = u.p;
    TORCH_CHECK(cosines.dim() == 4 && cosines.size(0) == p.F && cosines.size(1) == p.W && cosines.size(2) == p.S,
                "libhogatt: cosines must be [F, W, S, RotE]");
    TORCH_CHECK(sines.sizes() == cosines.sizes(), "libhogatt: sines must have the shape of cosines");
    TORCH_CHECK(cosines.scalar_type() == at::kFloat && sines.scalar_type() == at::kFloat, "libhogatt: cosines/sines must be float32");
    TORCH_CHECK(cosines.is_contiguous() && sines.is_contiguous(), "libhogatt: cosines/sines must be contiguous");
    TORCH_CHECK(rq.dim() == 5 && rq.size(0) == p.F && rq.size(1) == p.W && rq.size(2) == p.Hq && rq.size(3) == p.S && rq.size(4) == p.E,
                "libhogatt: rq must be [F, W, Hq, S, E]");
    TORCH_CHECK(rq.is_contiguous() && rq.scalar_type() == out.scalar_type(), "libhogatt: rq must be contiguous in the output dtype");
    u.p.RotE = (int32_t)cosines.size(3);
    u.p.cosines = cosines.const_data_ptr<float>();
    u.p.sines = sines.const_data_ptr<float>();
    u.p.rq = rq.data_ptr();
}

// ---- operators -------------------------------------------------------------------------------------------------

void hogwild_sdpa(at::Tensor& out, double scale, const at::Tensor& locations, const at::Tensor& queries,
                  const at::Tensor& fragment_lengths, const std::vector<at::Tensor>& key_fragments,
                  const std::vector<at::Tensor>& value_fragments) {
    Unpacked u;
    unpack_common(u, out, scale, locations, queries, fragment_lengths, key_fragments, value_fragments, true, false);
    run(u, out, false);
}

void hogwild_sdpa_lse(at::Tensor& out, at::Tensor& lse, double scale, const at::Tensor& locations, const at::Tensor& queries,
                      const at::Tensor& fragment_lengths, const std::vector<at::Tensor>& key_fragments,
                      const std::vector<at::Tensor>& value_fragments) {
    Unpacked u;
    unpack_common(u, out, scale, locations, queries, fragment_lengths, key_fragments, value_fragments, true, false);
    attach_lse(u, out, lse);
    run(u, out, false);
}

void hogwild_rope(at::Tensor& out, const at::Tensor& queries, const at::Tensor& cosines, const at::Tensor& sines) {
    TORCH_CHECK(out.dim() == 5 && queries.dim() == 4 && cosines.dim() == 4, "libhogatt: hogwild_rope expects out[F,W,Hq,S,E], "
                "queries[W,Hq,S,E], cosines/sines[F,W,S,RotE]");
    const int64_t F = out.size(0), W = out.size(1), Hq = out.size(2), S = out.size(3), E = out.size(4);
    TORCH_CHECK(queries.size(0) == W && queries.size(1) == Hq && queries.size(2) == S && queries.size(3) == E,
                "libhogatt: queries do not match the output shape");
    TORCH_CHECK(cosines.size(0) == F && cosines.size(1) == W && cosines.size(2) == S && sines.sizes() == cosines.sizes(),
                "libhogatt: cosines/sines do not match the output shape");
    TORCH_CHECK(out.is_contiguous() && queries.is_contiguous() && cosines.is_contiguous() && sines.is_contiguous(),
                "libhogatt: hogwild_rope needs contiguous tensors");
    TORCH_CHECK(queries.scalar_type() == out.scalar_type(), "libhogatt: queries and output must have the same dtype");
    TORCH_CHECK(cosines.scalar_type() == at::kFloat && sines.scalar_type() == at::kFloat, "libhogatt: cosines/sines must be float32");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(out.device());   // ROCm tensors report the device type "cuda"
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(out.device().index()).stream();
    check_status(hw_rope(out.data_ptr(), queries.const_data_ptr(), cosines.const_data_ptr<float>(), sines.const_data_ptr<float>(),
                         dtype_code(out), (int)F, (int)W, (int)Hq, (int)S, (int)E, (int)cosines.size(3), stream),
                 "hw_rope");
}

void hogwild_fused(at::Tensor& out, at::Tensor& rq, double scale, const at::Tensor& locations, const at::Tensor& queries,
                   const at::Tensor& fragment_lengths, const std::vector<at::Tensor>& key_fragments,
                   const std::vector<at::Tensor>& value_fragments, const at::Tensor& cosines, const at::Tensor& sines) {
    Unpacked u;
    unpack_common(u, out, scale, locations, queries, fragment_lengths, key_fragments, value_fragments, false, true);
    attach_rotation(u, out, rq, cosines, sines);
    run(u, out, true);
}

// Addition: the fused operator with `fragment_lengths` (int32 [F] in device memory) as the CURRENT lengths and the
// fragment tensors' sizes as bounds: fragment f has min(size, fragment_lengths[f]) tokens when the kernel runs, so a
// captured launch stays valid while segments grow inside their buffers.  (The reference reads the lengths from this
// tensor as well, src/kernels/kernel_v21.cuh:116-117, but needs them equal to the sizes.)
void hogwild_fused_devlen(at::Tensor& out, at::Tensor& rq, double scale, const at::Tensor& locations, const at::Tensor& queries,
                          const at::Tensor& fragment_lengths, const std::vector<at::Tensor>& key_fragments,
                          const std::vector<at::Tensor>& value_fragments, const at::Tensor& cosines, const at::Tensor& sines) {
    Unpacked u;
    unpack_common(u, out, scale, locations, queries, fragment_lengths, key_fragments, value_fragments, false, false);
    TORCH_CHECK(fragment_lengths.scalar_type() == at::kInt && fragment_lengths.is_contiguous() && fragment_lengths.device() == out.device(),
                "libhogatt: fragment_lengths must be contiguous int32 on the output's device");
    attach_rotation(u, out, rq, cosines, sines);
    u.p.len_dev = fragment_lengths.const_data_ptr<int32_t>();
    run(u, out, true);
}

void hogwild_fused_lse(at::Tensor& out, at::Tensor& rq, at::Tensor& lse, double scale, const at::Tensor& locations,
                       const at::Tensor& queries, const at::Tensor& fragment_lengths, const std::vector<at::Tensor>& key_fragments,
                       const std::vector<at::Tensor>& value_fragments, const at::Tensor& cosines, const at::Tensor& sines) {
    Unpacked u;
    unpack_common(u, out, scale, locations, queries, fragment_lengths, key_fragments, value_fragments, false, true);
    attach_rotation(u, out, rq, cosines, sines);
    attach_lse(u, out, lse);
    run(u, out, true);
}

// ---- paged operators -------------------------------------------------------------------------------------------

// Checks shared by the two paged attention operators; fills everything of hw_paged_problem except the query layout.
void unpack_paged(hw_paged_problem& p, at::Tensor& out, double scale, const at::Tensor& locations, const at::Tensor& queries,
                  const at::Tensor& fragment_lengths, const at::Tensor& key_cache, const at::Tensor& value_cache,
                  const at::Tensor& block_table) {
    TORCH_CHECK(key_cache.dim() == 4 && value_cache.dim() == 4, "libhogatt: caches must be [num_blocks, Hkv, block_size, D]");
    TORCH_CHECK(key_cache.size(0) == value_cache.size(0) && key_cache.size(1) == value_cache.size(1) && key_cache.size(2) == value_cache.size(2),
                "libhogatt: key_cache and value_cache differ in blocks, heads or block size");
    TORCH_CHECK(block_table.dim() == 2 && block_table.scalar_type() == at::kInt && block_table.is_contiguous(),
                "libhogatt: block_table must be contiguous int32 [W, max_blocks]");
    TORCH_CHECK(locations.scalar_type() == at::kInt && locations.is_contiguous(), "libhogatt: locations must be contiguous int32");
    TORCH_CHECK(fragment_lengths.scalar_type() == at::kInt && fragment_lengths.is_contiguous(), "libhogatt: fragment_lengths must be contiguous int32");
    TORCH_CHECK(out.is_contiguous() && queries.is_contiguous() && key_cache.is_contiguous() && value_cache.is_contiguous(),
                "libhogatt: output, queries and caches must be contiguous");
    TORCH_CHECK(queries.scalar_type() == out.scalar_type() && key_cache.scalar_type() == out.scalar_type() && value_cache.scalar_type() == out.scalar_type(),
                "libhogatt: queries and caches must have the dtype of the output");
    for (const at::Tensor* t : {&locations, &queries, &fragment_lengths, &key_cache, &value_cache, &block_table})
        TORCH_CHECK(t->device() == out.device(), "libhogatt: all tensors must live on the output's device");
    p.dtype = dtype_code(out);
    p.F = (int32_t)locations.size(0);
    p.W = (int32_t)block_table.size(0);
    p.Hkv = (int32_t)key_cache.size(1);
    p.E = (int32_t)key_cache.size(3);
    p.Ev = (int32_t)value_cache.size(3);
    p.block_size = (int32_t)key_cache.size(2);
    p.max_blocks = (int32_t)block_table.size(1);
    p.num_blocks = (int32_t)key_cache.size(0);
    p.scale = (float)scale;
    p.out = out.data_ptr();
    p.q = queries.const_data_ptr();
    p.locations = locations.const_data_ptr<int32_t>();
    p.fragment_lengths = fragment_lengths.const_data_ptr<int32_t>();
    p.key_cache = key_cache.const_data_ptr();
    p.value_cache = value_cache.const_data_ptr();
    p.block_table = block_table.const_data_ptr<int32_t>();
}

void run_paged(hw_paged_problem& p, const at::Tensor& out, bool varlen) {
    c10::hip::HIPGuardMasqueradingAsCUDA guard(out.device());
    size_t bytes = 0;
    check_status(hw_paged_workspace_bytes(&p, &bytes), "hw_paged_workspace_bytes");
    at::Tensor workspace = at::empty({(int64_t)(bytes > 0 ? bytes : 256)}, out.options().dtype(at::kByte));
    p.workspace = workspace.data_ptr();
    p.workspace_bytes = bytes;
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(out.device().index()).stream();
    if (varlen)
        check_status(hw_varlen_paged_sdpa(&p, stream), "hw_varlen_paged_sdpa");
    else
        check_status(hw_paged_sdpa(&p, stream), "hw_paged_sdpa");
}

void hogwild_paged_sdpa(at::Tensor& out, double scale, const at::Tensor& locations, const at::Tensor& queries,
                        const at::Tensor& fragment_lengths, const at::Tensor& key_cache, const at::Tensor& value_cache,
                        const at::Tensor& block_table) {
    hw_paged_problem p{};
    unpack_paged(p, out, scale, locations, queries, fragment_lengths, key_cache, value_cache, block_table);
    TORCH_CHECK(out.dim() == 4 && out.size(0) == p.W && out.size(3) == p.Ev, "libhogatt: output must be [W, Hq, S, Ev] with one block-table row per worker");
    p.Hq = (int32_t)out.size(1);
    p.S = (int32_t)out.size(2);
    TORCH_CHECK(queries.dim() == 5 && queries.size(0) == p.F && queries.size(1) == p.W && queries.size(2) == p.Hq && queries.size(3) == p.S && queries.size(4) == p.E,
                "libhogatt: queries must be [F, W, Hq, S, E]");
    TORCH_CHECK(locations.dim() == 3 && locations.size(1) == p.W && locations.size(2) == p.S, "libhogatt: locations must be [F, W, S]");
    TORCH_CHECK(fragment_lengths.dim() == 1 && fragment_lengths.size(0) == p.F, "libhogatt: fragment_lengths must be [F]");
    run_paged(p, out, false);
}

void hogwild_varlen_paged_sdpa(at::Tensor& out, double scale, const at::Tensor& locations, const at::Tensor& queries,
                               const at::Tensor& fragment_lengths, const at::Tensor& key_cache, const at::Tensor& value_cache,
                               const at::Tensor& block_table, const at::Tensor& cu_seqlens_q, const at::Tensor& cu_seqlens_k) {
    hw_paged_problem p{};
    unpack_paged(p, out, scale, locations, queries, fragment_lengths, key_cache, value_cache, block_table);
    TORCH_CHECK(out.dim() == 3 && out.size(2) == p.Ev, "libhogatt: output must be [total_q, Hq, Ev]");
    p.total_q = (int32_t)out.size(0);
    p.Hq = (int32_t)out.size(1);
    TORCH_CHECK(queries.dim() == 4 && queries.size(0) == p.F && queries.size(1) == p.total_q && queries.size(2) == p.Hq && queries.size(3) == p.E,
                "libhogatt: queries must be [F, total_q, Hq, E]");
    TORCH_CHECK(locations.dim() == 2 && locations.size(1) == p.total_q, "libhogatt: locations must be [F, total_q]");
    TORCH_CHECK(fragment_lengths.dim() == 2 && fragment_lengths.size(0) == p.F && fragment_lengths.size(1) == p.W,
                "libhogatt: fragment_lengths must be [F, W]");
    TORCH_CHECK(cu_seqlens_q.dim() == 1 && cu_seqlens_q.size(0) == p.W + 1 && cu_seqlens_q.scalar_type() == at::kInt &&
                    cu_seqlens_q.is_contiguous() && cu_seqlens_q.device() == out.device(),
                "libhogatt: cu_seqlens_q must be contiguous int32 [W + 1] on the output's device");
    (void)cu_seqlens_k;   // carried in the reference's Shape but never read by its kernel (src/kernels/kernel_v21.cuh:658-899)
    p.cu_seqlens_q = cu_seqlens_q.const_data_ptr<int32_t>();
    run_paged(p, out, true);
}

void copy_to_blocks(const at::Tensor& key_states, const at::Tensor& value_states, at::Tensor& key_cache, at::Tensor& value_cache,
                    const at::Tensor& block_table, const at::Tensor& seq_lengths) {
    TORCH_CHECK(key_states.dim() == 4 && value_states.dim() == 4, "libhogatt: key_states / value_states must be [B, Hkv, S_new, D]");
    TORCH_CHECK(key_states.size(0) == value_states.size(0) && key_states.size(1) == value_states.size(1) && key_states.size(2) == value_states.size(2),
                "libhogatt: key_states and value_states differ in batch, heads or tokens");
    TORCH_CHECK(key_cache.dim() == 4 && value_cache.dim() == 4 && key_cache.is_contiguous() && value_cache.is_contiguous(),
                "libhogatt: caches must be contiguous [num_blocks, Hkv, block_size, D]");
    TORCH_CHECK(key_cache.size(0) == value_cache.size(0) && key_cache.size(1) == key_states.size(1) && value_cache.size(1) == key_states.size(1) &&
                    key_cache.size(2) == value_cache.size(2) && key_cache.size(3) == key_states.size(3) && value_cache.size(3) == value_states.size(3),
                "libhogatt: caches do not match the states");
    TORCH_CHECK(value_states.scalar_type() == key_states.scalar_type() && key_cache.scalar_type() == key_states.scalar_type() &&
                    value_cache.scalar_type() == key_states.scalar_type(), "libhogatt: states and caches must share one dtype");
    TORCH_CHECK(block_table.dim() == 2 && block_table.size(0) == key_states.size(0) && block_table.scalar_type() == at::kInt && block_table.is_contiguous(),
                "libhogatt: block_table must be contiguous int32 [B, max_blocks]");
    TORCH_CHECK(seq_lengths.dim() == 1 && seq_lengths.size(0) == key_states.size(0) && seq_lengths.scalar_type() == at::kInt && seq_lengths.is_contiguous(),
                "libhogatt: seq_lengths must be contiguous int32 [B]");
    for (const at::Tensor* t : std::initializer_list<const at::Tensor*>{&key_states, &value_states, &value_cache, &block_table, &seq_lengths})
        TORCH_CHECK(t->device() == key_cache.device(), "libhogatt: all tensors must live on the caches' device");
    // any strides are fine as long as the head dimension is contiguous (the transposed view of a projection is)
    const at::Tensor ks = (key_states.size(3) > 1 && key_states.stride(3) != 1) ? key_states.contiguous() : key_states;
    const at::Tensor vs = (value_states.size(3) > 1 && value_states.stride(3) != 1) ? value_states.contiguous() : value_states;
    hw_copy_blocks c{};
    c.dtype = dtype_code(key_states);
    c.B = (int32_t)ks.size(0); c.Hkv = (int32_t)ks.size(1); c.S_new = (int32_t)ks.size(2);
    c.E = (int32_t)ks.size(3); c.Ev = (int32_t)vs.size(3);
    c.block_size = (int32_t)key_cache.size(2); c.max_blocks = (int32_t)block_table.size(1); c.num_blocks = (int32_t)key_cache.size(0);
    c.key_states = ks.const_data_ptr(); c.value_states = vs.const_data_ptr();
    c.ks_b = ks.stride(0); c.ks_h = ks.stride(1); c.ks_s = ks.stride(2);
    c.vs_b = vs.stride(0); c.vs_h = vs.stride(1); c.vs_s = vs.stride(2);
    c.key_cache = key_cache.data_ptr(); c.value_cache = value_cache.data_ptr();
    c.block_table = block_table.const_data_ptr<int32_t>(); c.seq_lengths = seq_lengths.const_data_ptr<int32_t>();
    c10::hip::HIPGuardMasqueradingAsCUDA guard(key_cache.device());
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(key_cache.device().index()).stream();
    check_status(hw_copy_to_blocks(&c, stream), "hw_copy_to_blocks");
}

}  // namespace

// `import hogatt` only has to load this shared object so that the registrations below run.
extern "C" PyObject* PyInit_hogatt(void) {
    static struct PyModuleDef def = {PyModuleDef_HEAD_INIT, "hogatt", "MI355X Hogwild! attention operators (namespace libhogatt)", -1, nullptr};
    return PyModule_Create(&def);
}

TORCH_LIBRARY(libhogatt, m) {
    const std::vector<at::Tag> tags = {at::Tag::needs_fixed_stride_order};
    m.def("hogwild_sdpa(Tensor(a!) output, float scale, Tensor locations, Tensor queries, "
          "Tensor fragment_lengths, Tensor[] key_fragments, Tensor[] value_fragments) -> ()", tags);
    m.def("hogwild_rope(Tensor(a!) output, Tensor queries, Tensor cosines, Tensor sines) -> ()", tags);
    m.def("hogwild_fused(Tensor(a!) output, Tensor(b!) rq, float scale, Tensor locations, Tensor queries, "
          "Tensor fragment_lengths, Tensor[] key_fragments, Tensor[] value_fragments, Tensor cosines, Tensor sines) -> ()", tags);
    // additions: same arguments plus the float32 [W, Hq, S] log-sum-exp output
    m.def("hogwild_sdpa_lse(Tensor(a!) output, Tensor(b!) lse, float scale, Tensor locations, Tensor queries, "
          "Tensor fragment_lengths, Tensor[] key_fragments, Tensor[] value_fragments) -> ()", tags);
    m.def("hogwild_fused_lse(Tensor(a!) output, Tensor(b!) rq, Tensor(c!) lse, float scale, Tensor locations, Tensor queries, "
          "Tensor fragment_lengths, Tensor[] key_fragments, Tensor[] value_fragments, Tensor cosines, Tensor sines) -> ()", tags);
    m.def("hogwild_fused_devlen(Tensor(a!) output, Tensor(b!) rq, float scale, Tensor locations, Tensor queries, "
          "Tensor fragment_lengths, Tensor[] key_fragments, Tensor[] value_fragments, Tensor cosines, Tensor sines) -> ()", tags);
    // the paged operators, schemas of src/binding.cu:369-374
    m.def("hogwild_paged_sdpa(Tensor(a!) output, float scale, Tensor locations, Tensor queries, "
          "Tensor fragment_lengths, Tensor key_cache, Tensor value_cache, Tensor block_table) -> ()", tags);
    m.def("copy_to_blocks(Tensor key_states, Tensor value_states, Tensor(a!) key_cache, Tensor(b!) value_cache, "
          "Tensor block_table, Tensor seq_lengths) -> ()", tags);
    m.def("hogwild_varlen_paged_sdpa(Tensor(a!) output, float scale, Tensor locations, Tensor queries, "
          "Tensor fragment_lengths, Tensor key_cache, Tensor value_cache, Tensor block_table, Tensor cu_seqlens_q, Tensor cu_seqlens_k) -> ()", tags);
}

TORCH_LIBRARY_IMPL(libhogatt, CUDA, m) {
    m.impl("hogwild_sdpa", hogwild_sdpa);
    m.impl("hogwild_rope", hogwild_rope);
    m.impl("hogwild_fused", hogwild_fused);
    m.impl("hogwild_sdpa_lse", hogwild_sdpa_lse);
    m.impl("hogwild_fused_lse", hogwild_fused_lse);
    m.impl("hogwild_fused_devlen", hogwild_fused_devlen);
    m.impl("hogwild_paged_sdpa", hogwild_paged_sdpa);
    m.impl("copy_to_blocks", copy_to_blocks);
    m.impl("hogwild_varlen_paged_sdpa", hogwild_varlen_paged_sdpa);
}
