// PyTorch operator binding for the MI355X Hogwild! attention library.
//
// Registers the operators of the reference's namespace `libhogatt` that lie on the fused decode path, with
// the same schema strings (src/binding.cu:363-367 of the reference), on the dispatch key ROCm tensors use
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
//   * `hogwild_fused_lse` / `hogwild_sdpa_lse` additionally return the log-sum-exp per query row.

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

struct Unpacked {
    hw_problem p{};
    std::vector<at::Tensor> keep;          // contiguous fragment tensors kept alive until the launch is queued
    std::vector<const void*> kptr, vptr;
    std::vector<int32_t> len;
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
        if (copy_noncontiguous) {   // the fused reference op does the same, src/binding.cu:330-337
            k = k.contiguous();
            v = v.contiguous();
        } else {
            TORCH_CHECK(k.is_contiguous() && v.is_contiguous(), "libhogatt: fragment ", f, " must be contiguous");
        }
        u.kptr[f] = k.const_data_ptr();
        u.vptr[f] = v.const_data_ptr();
        u.len[f] = (int32_t)k.size(1);
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
}

void run(Unpacked& u, const at::Tensor& out, bool fused) {
    c10::hip::HIPGuardMasqueradingAsCUDA guard(out.device());   // ROCm tensors report the device type "cuda"
    size_t bytes = 0;
    check_status(hw_workspace_bytes(&u.p, &bytes), "hw_workspace_bytes");
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

void hogwild_fused_lse(at::Tensor& out, at::Tensor& rq, at::Tensor& lse, double scale, const at::Tensor& locations,
                       const at::Tensor& queries, const at::Tensor& fragment_lengths, const std::vector<at::Tensor>& key_fragments,
                       const std::vector<at::Tensor>& value_fragments, const at::Tensor& cosines, const at::Tensor& sines) {
    Unpacked u;
    unpack_common(u, out, scale, locations, queries, fragment_lengths, key_fragments, value_fragments, false, true);
    attach_rotation(u, out, rq, cosines, sines);
    attach_lse(u, out, lse);
    run(u, out, true);
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
}

TORCH_LIBRARY_IMPL(libhogatt, CUDA, m) {
    m.impl("hogwild_sdpa", hogwild_sdpa);
    m.impl("hogwild_rope", hogwild_rope);
    m.impl("hogwild_fused", hogwild_fused);
    m.impl("hogwild_sdpa_lse", hogwild_sdpa_lse);
    m.impl("hogwild_fused_lse", hogwild_fused_lse);
}
