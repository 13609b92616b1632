/*
 * hogwild_hip.h — C ABI of the MI355X (gfx950) Hogwild! fragmented-KV attention library.
 *
 * This is the boundary a binding for the reference's operator API talks to: plain pointers and sizes,
 * no torch types, no C++ exceptions.  Every entry point returns 0 on success, a negative hw_status for
 * an argument / support error detected on the host (before any device work is queued), or a positive
 * hipError_t value if the HIP runtime reported one.
 *
 * Entry point  <->  reference interface it replaces (paths relative to the reference tree):
 *   hw_fused_attention ..... hogwild_fused            src/binding.cu:324-340 (schema :366-367)
 *   hw_sdpa ................ hogwild_attention        src/binding.cu:255-267, :39-108 (schema :363-364)
 *                            + launcher v21::hogwild_attention_gpu, src/kernels/kernel_v21.cuh:951-996
 *   hw_rope ................ hogwild_rope             src/binding.cu:298-308, :217-253; src/rope.cuh:54-62
 *   hw_workspace_bytes, hw_sdpa_workspace_bytes ... the launcher's private workspace sizing, src/kernels/kernel_v21.cuh:969-980
 *   hw_problem ............. struct Shape + the launcher argument list, src/common.h:5-20,
 *                            src/kernels/kernel_v21.cuh:951-957
 *   hw_status / hw_status_string ... cudaError_t + CUDA_RETURN_ON_ERROR, src/cuda_check.cuh:6-29
 *   hw_paged_sdpa .......... hogwild_paged_sdpa       src/binding.cu:110-142, :269-281 (schema :369-370)
 *                            + launcher v21::hogwild_paged_attention_gpu, src/kernels/kernel_v21.cuh:998-1043
 *   hw_varlen_paged_sdpa ... hogwild_varlen_paged_sdpa  src/binding.cu:144-181, :283-296 (schema :373-374)
 *                            + launcher v21::hogwild_varlen_paged_attention_gpu, src/kernels/kernel_v21.cuh:1045-1086
 *   hw_copy_to_blocks ...... copy_to_blocks           src/binding.cu:183-215, :310-322 (schema :371-372);
 *                            kernel src/cache.cuh:6-49
 *   hw_paged_problem ....... struct Shape with its paged / varlen members, src/common.h:5-20
 *   hw_build_inputs ........ the layer-0 branch of HogwildCache.update, python/hogwild/attention.py:164-196
 *                            (locations :173-181, model.rotary_emb + float cast :191-193)
 *   hw_rope_append ......... apply_rotary_pos_emb on the new keys + the per-worker cache update,
 *                            python/hogwild/attention.py:84-90, :313-318, :148-158; and merge_caches, :251-257
 *   hw_build_inputs_dev, hw_advance_lengths, hw_problem.len_dev, hw_append.len_dev ... no counterpart: the same steps
 *                            with the segment lengths in device memory, so that a decode step captured as a HIP graph
 *                            can be replayed while the segments grow
 */
#ifndef HOGWILD_HIP_H
#define HOGWILD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HW_ABI_VERSION 6
#define HW_MAX_FRAGMENTS 512          /* fragments per call, the reference's limit (src/binding.cu:79-82) */
#define HW_MAX_LAUNCH_FRAGMENTS 64    /* fragments one attention launch takes (their table travels in the kernel arguments);
                                         a call with more runs ceil(F / 64) attention launches, whose split-K partials lie
                                         side by side in the workspace, and one merge over all of them */
#define HW_MAX_SPLITS 256             /* workgroups per kv head and launch */

typedef enum hw_status {
    HW_OK = 0,
    HW_ERR_NULL = -1,          /* a required pointer is NULL */
    HW_ERR_DTYPE = -2,         /* dtype is not one of hw_dtype */
    HW_ERR_SHAPE = -3,         /* a dimension is non-positive or inconsistent (Hq % Hkv, RotE > E, odd RotE, a fragment
                                  whose kv-head slice reaches 2 GiB, scale not positive and finite, ...) */
    HW_ERR_UNSUPPORTED = -4,   /* shape is valid but no kernel is instantiated for it (never a silent no-op) */
    HW_ERR_FRAGMENTS = -5,     /* F < 1 or F > HW_MAX_FRAGMENTS (HW_MAX_LAUNCH_FRAGMENTS where stated) */
    HW_ERR_WORKSPACE = -6,     /* workspace NULL or smaller than hw_workspace_bytes() */
    HW_ERR_ALIGN = -7,         /* a device pointer is not 16-byte aligned */
    HW_ERR_NO_DEVICE = -8,     /* no usable HIP device */
    HW_ERR_STATIC_SCRATCH = -9 /* hw_fused_attention_static: the problem needs more than HW_STATIC_SCRATCH_BYTES */
} hw_status;

typedef enum hw_dtype { HW_F32 = 0, HW_F16 = 1, HW_BF16 = 2 } hw_dtype;

/*
 * One decode step of one layer.  W workers x S query tokens, Hq query heads sharing Hkv kv heads,
 * F KV fragments.  Device pointers unless stated otherwise; all tensors contiguous.
 *
 *   out        [W, Hq, S, Ev]      dtype     written
 *   lse        [W, Hq, S]          fp32      written if not NULL: ln sum_visible exp(scale * q.k); -inf for an empty row
 *   rq         [F, W, Hq, S, E]    dtype     hw_fused_attention only; written if not NULL (the rotated queries the
 *                                            reference materialises, src/binding.cu:338)
 *   q          hw_fused_attention: [W, Hq, S, E] un-rotated;  hw_sdpa: [F, W, Hq, S, E] already rotated
 *   locations  [F, W, S]           int32     query (w,s) sees key l of fragment f iff l <= locations[f,w,s]
 *                                            (src/kernels/kernel_v21.cuh:96-98)
 *   cosines, sines [F, W, S, RotE] fp32      hw_fused_attention only (src/rope.cuh:18-51 index convention)
 *   k, v       HOST arrays of F device pointers; fragment f is [Hkv, len[f], E] / [Hkv, len[f], Ev]
 *   len        HOST array of F lengths (the reference reads the same numbers from the tensor sizes, src/binding.cu:91)
 *   cap        optional HOST array of F row capacities: kv head h of fragment f starts h * cap[f] rows into its
 *              buffers (a segment that grows in place inside a [Hkv, cap, D] allocation).  NULL = packed, cap == len.
 *   len_dev    optional DEVICE array of F current lengths (hw_fused_attention with RotE == E only).  With it, len[f] is
 *              the bound the split is planned for and the buffers must hold (cap[f] >= len[f]), and fragment f has
 *              min(len[f], len_dev[f]) tokens when the kernel runs: a launch captured in a HIP graph stays valid while
 *              the segments grow up to len[f].  F <= HW_MAX_LAUNCH_FRAGMENTS.  No counterpart in the reference, whose
 *              segments are re-allocated by torch.cat on every update (python/hogwild/attention.py:148-158).
 *   workspace  device scratch of at least hw_workspace_bytes() bytes, caller-owned, 16-byte aligned
 *   splits     0 = choose automatically; otherwise the number of workgroups per kv head
 *   row_blocks 0 = choose automatically; 1 or 2 = 16-row MFMA blocks per workgroup (rows beyond that are
 *              spread over more workgroups that read the same KV); 8 = 128-row workgroups whose waves share every K/V
 *              tile through LDS (16-bit types without len_dev; the automatic choice beyond 96 rows per kv head)
 *   E, Ev      head dimensions: E == Ev in {64, 128, 256}, anything else returns HW_ERR_UNSUPPORTED (the reference's
 *              kernel is a template over E and Ev and is instantiated for 128 only, src/kernels/kernel_v21.cuh:28,982).
 *              Head dimension 256 exists with one 16-row block per workgroup (row_blocks is taken as 1) and without
 *              the VALU-logits variant; the paged operators take it in the 16-bit types.
 *   variant    HW_VARIANT_MFMA (0, default): logits and output on the matrix cores.  HW_VARIANT_VALU_QK: the logits
 *              K.Q^T by VALU dot products (v_dot2_f32_bf16 / _f16, v_fma_f32) in the same kernel, the inner product the
 *              reference uses (src/kernels/kernel_v21.cuh:161-180); exists so that the matrix-core choice can be measured
 *              for workloads with at most 16 query rows per kv head (hw_fused_attention, RotE == E, host lengths;
 *              anything else returns HW_ERR_UNSUPPORTED).
 */
#define HW_VARIANT_MFMA 0
#define HW_VARIANT_VALU_QK 1
typedef struct hw_problem {
    int32_t dtype;
    int32_t F, W, Hq, Hkv, S, E, Ev, RotE;
    float scale;
    void* out;
    float* lse;
    void* rq;
    const void* q;
    const int32_t* locations;
    const float* cosines;
    const float* sines;
    const void* const* k;
    const void* const* v;
    const int32_t* len;
    void* workspace;
    size_t workspace_bytes;
    int32_t splits;
    int32_t row_blocks;
    const int32_t* cap;
    const int32_t* len_dev;
    int32_t variant;
} hw_problem;

/* How a problem is cut into workgroups; filled by hw_plan_debug (host only, no device needed). */
typedef struct hw_plan {
    int32_t rows;             /* W*S*(Hq/Hkv): query rows that share one kv head */
    int32_t row_blocks;       /* 16-row MFMA blocks per workgroup (1, 2 or 8) */
    int32_t row_groups;       /* workgroups along the row dimension */
    int32_t tile_tokens;      /* tokens per wave step */
    int32_t tiles_per_head;   /* sum_f ceil(len[f] / tile_tokens) */
    int32_t wgs_per_head;     /* split-K factor */
    int32_t workgroups;       /* grid size of the attention kernel */
    int32_t tile_begin[HW_MAX_LAUNCH_FRAGMENTS + 1];   /* first tile of each fragment in a head's tile sequence */
    int32_t wg_tile_begin[HW_MAX_SPLITS + 1];   /* first tile of each workgroup; balanced by tiles + a fixed
                                                    cost for every fragment a workgroup has to open */
    size_t workspace_bytes;
} hw_plan;

int hw_version(void);
const char* hw_status_string(int status);

/* Host-only argument check shared by all entry points (pointer checks cover what `fused` != 0 needs). */
int hw_validate(const hw_problem* p, int fused);

/* Host-only: the split plan of one attention launch for a device with `num_cus` compute units
   (F <= HW_MAX_LAUNCH_FRAGMENTS; a call with more fragments plans each group of 64 like this). */
int hw_plan_debug(const hw_problem* p, int num_cus, hw_plan* plan);

/* Workspace size for the current device: what hw_fused_attention needs for this problem (if the rotary width is not
   the head dimension and p->rq is NULL, that includes room for the rotated queries); enough for hw_sdpa as well. */
int hw_workspace_bytes(const hw_problem* p, size_t* bytes);
/* The same for hw_sdpa alone (pre-rotated queries: RotE, cosines, sines and rq are ignored). */
int hw_sdpa_workspace_bytes(const hw_problem* p, size_t* bytes);

/* Rotate q per fragment in registers and attend; replaces hogwild_fused. */
int hw_fused_attention(const hw_problem* p, void* stream);

/*
 * hw_fused_attention for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same inputs, outputs and kernels as
 * hw_fused_attention, except that p->workspace / p->workspace_bytes are ignored: the split-K partials go to a
 * device array that is part of the library image (HW_STATIC_SCRATCH_BYTES per GPU, resident until the process ends).
 * The call allocates and frees nothing.  A problem whose hw_workspace_bytes() exceeds HW_STATIC_SCRATCH_BYTES is
 * refused with HW_ERR_STATIC_SCRATCH before anything is queued -- except that with row_blocks = 0 a plan of 128-row
 * workgroups that does not fit is replaced by the 32-row kernel's (fewer partials), and only that one has to fit.  All calls on one GPU share that GPU's array: calls
 * that overlap in time on one GPU (different streams, or graphs replayed concurrently) race on the partials and
 * must be serialised by the caller.  Nothing in the array has to survive between calls or start at zero.
 */
#define HW_STATIC_SCRATCH_BYTES (8u << 20)
int hw_fused_attention_static(const hw_problem* p, void* stream);

/* The two kernels of hw_fused_attention separately.  HW_STAGE_ATTENTION leaves the split-K partials of this
   device's KV in the workspace (per kv head and workgroup: unnormalised output rows, running max in base-2 units
   and sum); HW_STAGE_MERGE combines the partials found there into out / lse.  For a caller that holds only part of
   the fragments and exchanges partials before merging, and for timing the attention kernel alone.  The reference
   has the same split internally (kernel + reduce kernel, src/kernels/kernel_v21.cuh:985-989). */
#define HW_STAGE_ATTENTION 1
#define HW_STAGE_MERGE 2
int hw_fused_attention_stages(const hw_problem* p, void* stream, int stages);

/* Attend with already-rotated queries [F,W,Hq,S,E]; replaces hogwild_sdpa. */
int hw_sdpa(const hw_problem* p, void* stream);

/* out[F,W,Hq,S,E] = rope(q[W,Hq,S,E], cos/sin[F,W,S,RotE]); replaces hogwild_rope. */
int hw_rope(void* out, const void* q, const float* cosines, const float* sines, int dtype,
            int F, int W, int Hq, int S, int E, int RotE, void* stream);

/* ------------------------------------------------------------------------------------------------------------
 * Paged variants: the KV of worker (sequence) w lives in blocks of one cache tensor and is found through a block
 * table (src/kernels/kernel_v21.cuh:405-411).  Every fragment f attends the same sequence from position 0 with its
 * own queries and its own bound min(fragment_lengths, location + 1) (kernel_v21.cuh:385-388).
 *
 *   key_cache   [num_blocks, Hkv, block_size, E]    dtype
 *   value_cache [num_blocks, Hkv, block_size, Ev]   dtype
 *   block_table [W, max_blocks]                     int32; position l of sequence w is row l % block_size of block
 *                                                   block_table[w][l / block_size].  Entries are clamped into
 *                                                   0..num_blocks-1 on the device (a corrupt table reads wrong rows
 *                                                   but never outside the cache).
 * fixed-length operator (cu_seqlens_q == NULL), hw_paged_sdpa:
 *   q [F, W, Hq, S, E] rotated, locations [F, W, S], fragment_lengths [F] (device), out [W, Hq, S, Ev], lse [W, Hq, S]
 * packed variable-length operator (cu_seqlens_q != NULL), hw_varlen_paged_sdpa:
 *   q [F, total_q, Hq, E] rotated, locations [F, total_q], fragment_lengths [F, W] (device), cu_seqlens_q [W + 1]
 *   (device; query tokens cu[w] .. cu[w+1]-1 belong to sequence w, kernel_v21.cuh:15-23), out [total_q, Hq, Ev],
 *   lse [total_q, Hq].  S is ignored.
 * Nothing is read from a sequence beyond what some query row can see, so the lengths need not be known on the host.
 * Limits: block_size < 4096, block_size * max_blocks <= 2^20 positions per sequence, num_blocks * Hkv * block_size
 * < 2^31 cache rows, query rows per kv head (tokens * Hq/Hkv) < 2^20.
 */
typedef struct hw_paged_problem {
    int32_t dtype;
    int32_t F, W, Hq, Hkv, E, Ev;
    int32_t S;                 /* query tokens per worker (fixed-length operator) */
    int32_t total_q;           /* packed query tokens over all workers (variable-length operator) */
    int32_t block_size, max_blocks, num_blocks;
    float scale;
    void* out;
    float* lse;                /* optional */
    const void* q;
    const int32_t* locations;
    const int32_t* fragment_lengths;
    const void* key_cache;
    const void* value_cache;
    const int32_t* block_table;
    const int32_t* cu_seqlens_q;   /* NULL selects the fixed-length operator */
    void* workspace;
    size_t workspace_bytes;
    int32_t splits;            /* 0 = automatic (packed queries in 128-row workgroups: decided on the device, see
                                  hw_paged_plan.device_planned); otherwise workgroups per (kv head, row group) */
    int32_t row_blocks;        /* 0 = automatic; 1, 2 or 8 = 16-row MFMA blocks per workgroup (8: workgroups of up to 128 rows
                                  whose waves share every K/V tile, 16-bit types, max_blocks <= 8192; the automatic choice
                                  beyond 16 query rows per sequence and kv head -- for packed queries, whose lengths are
                                  device data, beyond 16 on average over the sequences) */
} hw_paged_problem;

typedef struct hw_paged_plan {
    int32_t rows;              /* query rows per kv head: tokens * Hq/Hkv */
    int32_t row_blocks;
    int32_t row_groups;        /* over all workers; an upper bound for the variable-length operator */
    int32_t splits;            /* workgroups per (kv head, row group); tile t of a sequence goes to wave t mod (4 * splits) */
    int32_t workgroups;
    int32_t device_planned;    /* packed queries in 128-row workgroups: the split is decided on the device from the query and KV
                                  lengths, in the prologue of the attention kernel.  row_groups is then the number
                                  of workgroup slots per kv head (each takes a row group's share of tiles, or nothing),
                                  splits = 1 */
    size_t workspace_bytes;
} hw_paged_plan;

int hw_paged_validate(const hw_paged_problem* p);
int hw_paged_plan_debug(const hw_paged_problem* p, int num_cus, hw_paged_plan* plan);   /* host only */
int hw_paged_workspace_bytes(const hw_paged_problem* p, size_t* bytes);
/* replaces hogwild_paged_sdpa (cu_seqlens_q must be NULL) */
int hw_paged_sdpa(const hw_paged_problem* p, void* stream);
/* replaces hogwild_varlen_paged_sdpa (cu_seqlens_q must not be NULL) */
int hw_varlen_paged_sdpa(const hw_paged_problem* p, void* stream);
/* either operator, attention kernel and merge kernel separately (HW_STAGE_*), for timing */
int hw_paged_sdpa_stages(const hw_paged_problem* p, void* stream, int stages);

/*
 * Append new K/V rows to the paged caches: token t of sequence b goes to position seq_lengths[b] + t of that
 * sequence (src/cache.cuh:29-48).  key_states / value_states are [B, Hkv, S_new, E|Ev] with element strides
 * (ks_*, vs_*) for the first three dimensions and a contiguous last dimension, so the usual transposed view of a
 * [B, S_new, Hkv, D] projection can be passed as it is.  block_table [B, max_blocks], seq_lengths [B]: device int32.
 * A position outside the block table, or a table entry outside the cache, is skipped (the reference would write out
 * of bounds).  The reference launches S_new * max(E, Ev) threads per block and therefore cannot take more than
 * 8 new tokens at head dimension 128 (src/binding.cu:201-203); there is no such limit here.
 */
typedef struct hw_copy_blocks {
    int32_t dtype;
    int32_t B, Hkv, S_new, E, Ev;
    int32_t block_size, max_blocks, num_blocks;
    const void* key_states;
    const void* value_states;
    int64_t ks_b, ks_h, ks_s;
    int64_t vs_b, vs_h, vs_s;
    void* key_cache;
    void* value_cache;
    const int32_t* block_table;
    const int32_t* seq_lengths;
} hw_copy_blocks;

int hw_copy_to_blocks(const hw_copy_blocks* c, void* stream);

/* ------------------------------------------------------------------------------------------------------------
 * Caller-side steps of a decode step (the reference does them in Python, python/hogwild/attention.py:137-204,251-257).
 */

/*
 * locations[f,w,s] = pos_end[f*W + w] - S + s and the query rotation tables of those positions:
 * cos/sin[f,w,s,i] = cos/sin(float(location) * inv_freq[i mod RotE/2]) * attention_scaling, fp32 arithmetic, rounded to
 * `round_dtype` (HW_F32 = no rounding; the model library hands out the tables in the model dtype and the reference
 * widens them back to fp32, python/hogwild/attention.py:191-193) and stored as fp32.
 *   pos_end    HOST array [F, W]: for fragment f and worker w, the sum of the lengths of f and of every fragment that
 *              follows f in worker w's order, new tokens included (python/hogwild/attention.py:174-181)
 *   inv_freq   device fp32 [RotE/2]
 *   locations  device int32 [F, W, S]; cosines / sines device fp32 [F, W, S, RotE]
 */
int hw_build_inputs(int32_t* locations, float* cosines, float* sines, const int32_t* pos_end, const float* inv_freq,
                    float attention_scaling, int round_dtype, int F, int W, int S, int RotE, void* stream);

/*
 * The same with the lengths in device memory, for decode steps replayed from a HIP graph: pos_end[f][w] is formed in
 * the kernel as the sum of len_dev over fragment f and everything behind it in worker w's order.
 *   len_dev    device int32 [F]: current fragment lengths (including this step's new tokens)
 *   orders     HOST int32 [W, F]: orders[w][i] = the i-th fragment of worker w's order (every fragment once)
 * F * W <= 768.
 */
int hw_build_inputs_dev(int32_t* locations, float* cosines, float* sines, const int32_t* len_dev, const int32_t* orders,
                        const float* inv_freq, float attention_scaling, int round_dtype, int F, int W, int S, int RotE,
                        void* stream);

/* len_dev[f] += add[f] for f < F <= HW_MAX_LAUNCH_FRAGMENTS (add is a HOST array): the first node of a captured decode step. */
int hw_advance_lengths(int32_t* len_dev, const int32_t* add, int F, void* stream);

#define HW_ROPE_EAGER 0   /* every product and the sum rounded as an eager tensor expression rounds them: bit-identical to
                             apply_rotary_pos_emb of the reference on the same dtypes */
#define HW_ROPE_FUSED 1   /* fp32 fused multiply-add, one rounding at the end */

/*
 * Rotate new keys and append keys and values to each worker's segment, in place:
 *   K_dst[w][h, len[w] + t, :] = rope(key_states[w, h, S - n_new[w] + t, :], cos/sin[w, S - n_new[w] + t, :])
 *   V_dst[w][h, len[w] + t, :] = value_states[w, h, S - n_new[w] + t, :]            t = 0 .. n_new[w]-1
 * (left masking, python/hogwild/attention.py:149-155).  rope = (x * cos) + (rotate_half(x) * sin) on the first RotE
 * elements, every element reading cos/sin at its own index (python/hogwild/attention.py:77-90); RotE == 0 appends
 * without rotating (keys that arrive rotated).  Device pointers unless stated otherwise.
 *   key_states / value_states   [W, Hkv, S, E|Ev] with element strides for the first three dimensions
 *   cosines / sines             [W, S, RotE] with element strides cs_w, cs_s, in fp32 (cs_dtype == HW_F32) or in `dtype`
 *                               (cs_dtype == dtype); cs_s == 0 applies one row to every token (merge_caches,
 *                               python/hogwild/attention.py:252-256)
 *   k_dst / v_dst               HOST arrays of W device pointers to segment buffers [Hkv, cap[w], E|Ev]
 *   dst_len / dst_cap / n_new   HOST arrays of W ints; len + n_new <= cap is checked on the host
 *   len_dev                     optional DEVICE int32 array of segment lengths.  With it dst_len[w] is an index into it,
 *                               len_dev[dst_len[w]] is the length of worker w's segment AFTER this append (rows already
 *                               there = that minus n_new[w]), and an append that would not fit dst_cap[w] is dropped.
 */
typedef struct hw_append {
    int32_t dtype, cs_dtype, mode;
    int32_t W, Hkv, S, E, Ev, RotE;
    const void* key_states;
    const void* value_states;
    int64_t ks_w, ks_h, ks_s;
    int64_t vs_w, vs_h, vs_s;
    const void* cosines;
    const void* sines;
    int64_t cs_w, cs_s;
    void* const* k_dst;
    void* const* v_dst;
    const int32_t* dst_len;
    const int32_t* dst_cap;
    const int32_t* n_new;
    const int32_t* len_dev;
} hw_append;

int hw_rope_append(const hw_append* a, void* stream);

/* Number of compute units of the current device (0 on failure). */
int hw_device_cus(void);

#ifdef __cplusplus
}
#endif
#endif /* HOGWILD_HIP_H */
