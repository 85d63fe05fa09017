/*
 * pie_driver_abi.h — the Pie runtime <-> driver boundary as this driver sees it.
 *
 * The Pie runtime hands an in-process driver plain-old-data descriptors through a
 * three-slot vtable (recv / send_response / ctx) and expects two exported symbols per
 * driver flavour.  This header re-states that C ABI for the `hip` flavour.  It is
 * written independently but is layout-compatible, field for field, with the
 * reference's driver/bridge/include/pie_bridge.h:250-451: every Rust `Vec<T>` is a
 * (pointer, size_t length) pair — expressed here as a two-member slice struct, which
 * has the same size, alignment and member offsets as the two loose fields — and
 * tagged enums are a kind byte followed by every variant's struct (not a union).
 * tests/test_abi_layout.py checks sizeof/offsetof of every struct against the
 * reference header when the reference tree is present.
 *
 * Ownership (driver/bridge/src/ffi.rs:19-34): a request descriptor and all slices in
 * it are borrowed from the runtime until send_response(req_id) is called and must not
 * be written; a response descriptor's slices are owned by the driver and must stay
 * valid until send_response returns.
 */
#ifndef PIE_DRIVER_ABI_H
#define PIE_DRIVER_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- slices ------------------------------------------------------------------- */
typedef struct PieU8Slice  { const uint8_t*  ptr; size_t len; } PieU8Slice;
typedef struct PieU32Slice { const uint32_t* ptr; size_t len; } PieU32Slice;
typedef struct PieU64Slice { const uint64_t* ptr; size_t len; } PieU64Slice;
typedef struct PieF32Slice { const float*    ptr; size_t len; } PieF32Slice;

/* ---- discriminants (pie_bridge.h:64-97) ------------------------------------------ */
enum { PIE_REQ_FORWARD = 0, PIE_REQ_COPY = 1, PIE_REQ_ADAPTER = 2, PIE_REQ_HEALTH = 3 };
enum { PIE_RESP_FORWARD = 0, PIE_RESP_STATUS = 1 };
enum {
    PIE_SAMPLER_KIND_MULTINOMIAL = 0, PIE_SAMPLER_KIND_TOP_K = 1, PIE_SAMPLER_KIND_TOP_P = 2,
    PIE_SAMPLER_KIND_MIN_P = 3, PIE_SAMPLER_KIND_TOP_K_TOP_P = 4, PIE_SAMPLER_KIND_EMBEDDING = 5,
    PIE_SAMPLER_KIND_DIST = 6, PIE_SAMPLER_KIND_RAW_LOGITS = 7, PIE_SAMPLER_KIND_LOGPROB = 8,
    PIE_SAMPLER_KIND_LOGPROBS = 9, PIE_SAMPLER_KIND_ENTROPY = 10
};
enum { PIE_COPY_D2H = 0, PIE_COPY_H2D = 1, PIE_COPY_D2D = 2, PIE_COPY_H2H = 3 };
enum { PIE_RESOURCE_KV = 0, PIE_RESOURCE_RS = 1 };
enum { PIE_ADAPTER_LOAD = 0, PIE_ADAPTER_SAVE = 1, PIE_ADAPTER_ZO_INIT = 2,
       PIE_ADAPTER_ZO_UPDATE = 3, PIE_ADAPTER_GENERATE_AUDIO = 4 };

/* Method tags a driver dispatches on, synthesised from payload kind + sub-op
 * (driver/bridge/include/pie_bridge/view.hpp:89-107,552-591). */
enum {
    PIE_METHOD_FORWARD = 0,
    PIE_METHOD_COPY_KV_D2H = 1, PIE_METHOD_COPY_KV_H2D = 2, PIE_METHOD_COPY_KV_D2D = 3,
    PIE_METHOD_COPY_KV_H2H = 4,
    PIE_METHOD_ADAPTER_LOAD = 5, PIE_METHOD_ADAPTER_SAVE = 6, PIE_METHOD_ADAPTER_ZO_INIT = 7,
    PIE_METHOD_ADAPTER_ZO_UPDATE = 8,
    PIE_METHOD_HEALTH = 9,
    PIE_METHOD_COPY_RS_D2H = 10, PIE_METHOD_COPY_RS_H2D = 11, PIE_METHOD_COPY_RS_D2D = 12,
    PIE_METHOD_COPY_RS_H2H = 13,
    PIE_METHOD_GENERATE_AUDIO = 14
};
#define PIE_METHOD_UNKNOWN 0xFFFFFFFFu

/* Status codes of non-forward replies
 * (driver/portable/src/service/inproc_service.cpp:82-203). */
enum { PIE_STATUS_OK = 0, PIE_STATUS_UNKNOWN_METHOD = 2, PIE_STATUS_OUT_OF_RANGE = 3,
       PIE_STATUS_UNSUPPORTED = 4, PIE_STATUS_FAILED = 5, PIE_STATUS_EXCEPTION = -1 };

/* ---- request side ------------------------------------------------------------- */
typedef struct PieAdapterBindingDesc {
    int64_t adapter_id; /* -1 = unbound */
    int64_t seed;       /* -1 = none given */
} PieAdapterBindingDesc;

/* Binary run-length mask: alternating run lengths (first run = false), total_size bits. */
typedef struct PieBrleDesc {
    PieU32Slice buffer;
    uint64_t total_size;
} PieBrleDesc;
typedef struct PieBrleSlice { const PieBrleDesc* ptr; size_t len; } PieBrleSlice;

typedef struct PieSamplerDesc {
    uint8_t kind;
    float temperature;
    uint32_t seed;
    uint32_t k;
    float p;
    uint32_t num_tokens;
    uint32_t token_id;
    PieU32Slice token_ids;
} PieSamplerDesc;
typedef struct PieSamplerSlice { const PieSamplerDesc* ptr; size_t len; } PieSamplerSlice;
typedef struct PieAdapterBindingSlice { const PieAdapterBindingDesc* ptr; size_t len; } PieAdapterBindingSlice;

typedef struct PieForwardRequestDesc {
    PieU32Slice token_ids;          /* [N] all requests' new tokens, concatenated       */
    PieU32Slice position_ids;       /* [N]                                              */
    PieU32Slice kv_page_indices;    /* concatenated physical page ids                   */
    PieU32Slice kv_page_indptr;     /* [R+1]                                            */
    PieU32Slice kv_last_page_lens;  /* [R] valid slots in each request's last page      */
    PieU32Slice qo_indptr;          /* [R+1] token rows of each request                 */
    PieU32Slice rs_slot_ids;
    PieU8Slice rs_slot_flags;
    PieBrleSlice masks;             /* per-token attention masks (may be empty)         */
    PieU32Slice mask_indptr;
    PieBrleSlice logit_masks;
    PieU32Slice logit_mask_indptr;
    PieU32Slice sampling_indices;   /* request-relative token rows to sample from       */
    PieU32Slice sampling_indptr;    /* [R+1]                                            */
    PieSamplerSlice samplers;
    PieU32Slice sampler_indptr;
    PieAdapterBindingSlice adapter_bindings;
    PieU32Slice spec_token_ids;
    PieU32Slice spec_position_ids;
    PieU32Slice spec_indptr;
    PieU8Slice output_spec_flags;
    PieU64Slice context_ids;
    uint8_t single_token_mode;
    uint8_t has_user_mask;
    /* multimodal spans: carried, unused by this driver */
    PieU32Slice image_indptr;
    PieU32Slice image_grids;
    PieU32Slice image_anchor_positions;
    PieU8Slice image_pixels;
    PieU32Slice image_pixel_indptr;
    PieU32Slice image_mrope_positions;
    PieU32Slice image_mrope_indptr;
    PieU32Slice image_patch_positions;
    PieU32Slice image_anchor_rows;
    PieU8Slice audio_features;
    PieU32Slice audio_feature_indptr;
    PieU32Slice audio_anchor_rows;
    PieU32Slice audio_indptr;
} PieForwardRequestDesc;

typedef struct PieCopyRequestDesc {
    uint8_t dir;
    PieU32Slice srcs;
    PieU32Slice dsts;
    uint8_t resource;
} PieCopyRequestDesc;

typedef struct PieAdapterRequestDesc {
    uint8_t op;
    uint64_t adapter_id;
    PieU8Slice path;
} PieAdapterRequestDesc;

typedef struct PieRequestPayloadDesc {
    uint8_t kind;
    PieForwardRequestDesc forward;
    PieCopyRequestDesc copy;
    PieAdapterRequestDesc adapter;
} PieRequestPayloadDesc;

typedef struct PieFrameDesc {
    uint32_t driver_id;
    PieRequestPayloadDesc payload;
} PieFrameDesc;

/* ---- response side ------------------------------------------------------------ */
typedef struct PieForwardResponseDesc {
    uint32_t num_requests;
    PieU32Slice tokens_indptr;       /* [R+1] */
    PieU32Slice tokens;
    PieU32Slice dists_req_indptr;    /* [R+1] */
    PieU32Slice dists_kv_indptr;     /* leading 0, one entry per dist */
    PieU32Slice dists_ids;
    PieF32Slice dists_probs;
    PieU32Slice logits_req_indptr;   /* [R+1] */
    PieU32Slice logits_byte_indptr;
    PieU8Slice logits_bytes;
    PieU32Slice logprobs_req_indptr; /* [R+1] */
    PieU32Slice logprobs_val_indptr;
    PieF32Slice logprobs_values;
    PieU32Slice entropies_indptr;    /* [R+1] */
    PieF32Slice entropies;
    PieU32Slice spec_indptr;         /* [R+1] */
    PieU32Slice spec_tokens;
    PieU32Slice spec_positions;
    uint32_t probe_wire_parse_us;
    uint32_t probe_plan_us;
    uint32_t probe_h2d_us;
    uint32_t probe_kernel_launch_us;
    uint32_t probe_sync_us;
    uint32_t probe_response_build_us;
} PieForwardResponseDesc;

typedef struct PieStatusResponseDesc {
    int32_t status;
} PieStatusResponseDesc;

typedef struct PieResponsePayloadDesc {
    uint8_t kind;
    PieForwardResponseDesc forward;
    PieStatusResponseDesc status;
} PieResponsePayloadDesc;

typedef struct PieResponseFrameDesc {
    uint32_t driver_id;
    uint8_t aborted;
    PieResponsePayloadDesc payload;
} PieResponseFrameDesc;

/* ---- in-process vtable (pie_bridge.h:427-451) ------------------------------------ */
/* recv blocks; 0 = a request is ready, -1 = clean shutdown, anything else = error. */
typedef struct PieInProcVTable {
    int32_t (*recv)(void* ctx, const PieFrameDesc** out_request, uint32_t* out_req_id);
    void (*send_response)(void* ctx, uint32_t req_id, const PieResponseFrameDesc* response);
    void* ctx;
} PieInProcVTable;

/* ---- exported driver entry points ------------------------------------------------- */
/*
 * Runs the driver on the calling thread until recv reports shutdown or request_stop is
 * called.  argv: program name, then `--config <file.toml>` (also `-c`, `--config=`).
 * ready_cb is called exactly once, after weights and the KV pool are allocated, with the
 * capabilities JSON (driver/bridge/src/capabilities.rs:18-78).  Returns 0, or -1 on any
 * failure; never lets a C++ exception cross the boundary.
 * Replaces pie_driver_portable_run_inproc (driver/portable/src/entry.cpp:483-498) as bound
 * by server/src/driver_ffi.rs:18-46.
 */
int pie_driver_hip_run_inproc(int argc, char** argv, int install_signal_handlers,
                              void (*ready_cb)(const char* caps_json, void* ctx),
                              void* ready_ctx, PieInProcVTable vtable);
/* Process-global stop for every live instance (driver/portable/src/entry.cpp:500-505): may be
 * called from any thread.  An instance registers on entry to run_inproc, before it loads its
 * model, so a stop requested while it loads makes it return (0) right after the ready
 * handshake without serving; a serving instance leaves its loop when the recv in progress
 * returns (recv may report "nothing yet" by returning 0 with a null frame). */
void pie_driver_hip_request_stop(void);

/* ---- direct (no vtable thread) embedding API ------------------------------------ */
/*
 * The same driver object the serve loop drives, for harnesses that call it synchronously:
 * create from a TOML config (a path, or inline text when it contains a newline), feed
 * frames, read the response until the next call.  Mirrors the offline self-test harness of
 * the reference (driver/portable/src/entry.cpp:252-263,387-409; Executor::generate_multi,
 * driver/portable/src/executor/executor.cpp:1439-1597).
 */
typedef struct PieHipDriver PieHipDriver;
PieHipDriver* pie_hip_driver_create(const char* config_toml, char* err, size_t err_cap);
void pie_hip_driver_destroy(PieHipDriver* d);
/* Capabilities JSON, valid for the driver's lifetime. */
const char* pie_hip_driver_capabilities(const PieHipDriver* d);
/* Handle one frame; *out stays valid until the next call on this driver.  Returns 0. */
int pie_hip_driver_handle(PieHipDriver* d, const PieFrameDesc* frame, PieResponseFrameDesc* out);
/*
 * Greedy generation harness: `replicate` independent contexts, each prefilled with the same
 * prompt on contiguous page ranges, then `max_new` single-token decode steps over all of
 * them in one forward per step.  out_tokens: [replicate, max_new].  The first `warmup`
 * decode steps are excluded from the decode timings.  timings_us (optional, 4 entries):
 * prefill wall, timed decode wall, timed decode device time (HIP events), steps timed.
 * Returns 0 or a negative error (message in err).
 */
int pie_hip_driver_generate(PieHipDriver* d, const uint32_t* prompt, int n_prompt, int max_new,
                            int replicate, int warmup, uint32_t* out_tokens, double* timings_us,
                            char* err, size_t err_cap);
/* Sampler the generation harness attaches to its decode steps instead of greedy: a wire kind
 * 0..4 (Multinomial, TopK, TopP, MinP, TopKTopP) with its fields; the seed is advanced per step
 * and context.  Returns 0, -1 on a bad kind. */
int pie_hip_driver_set_generate_sampler(PieHipDriver* d, int kind, float temperature, uint32_t k,
                                        float p, uint32_t seed);
/* Generation harness only (no counterpart in the reference): with stride > 0 replica c of
 * pie_hip_driver_generate feeds (its last sampled token + c * stride) % vocab into every decode
 * step, so the rows of a decode batch differ (distinct MoE routes); 0 (default) keeps identical
 * replicas. */
int pie_hip_driver_set_generate_divergence(PieHipDriver* d, uint32_t stride);
/* Host-only: what the snapshot reader sees in a Hugging Face checkpoint directory, as JSON
 * {"arch", shape fields, "tensors": {name: {"dtype", "shape", "bytes", "first_bytes"}}} written
 * to out.  Returns its length, or -1 with the reader's message in err.  No GPU is touched. */
long long pie_hip_driver_snapshot_info(const char* dir, char* out, size_t out_cap, char* err,
                                       size_t err_cap);
/* Copy a named tensor to host memory (test/bench hook): model weights by name, "kv.k.<l>" /
 * "kv.v.<l>" (layer l's page pool), "debug.logits" (last forward's sampled-row logits) and
 * row 0 of the last layer's intermediates of the last forward: "debug.q" (rotated queries,
 * q_heads * head_dim bf16), "debug.attn" (attention output), "debug.act" (SwiGLU output) and
 * "debug.x" (residual stream after the layer); "info.qk_rows_paired" / "info.rope_interleaved"
 * (one int32 each: whether wqkv's q / k rows are stored pair-interleaved, and the RoPE pairing).
 * Returns the byte size, 0 if the tensor does not exist; copies min(size, cap) bytes when dst
 * is non-null. */
size_t pie_hip_driver_export_tensor(PieHipDriver* d, const char* name, void* dst, size_t cap);
/* Device address of a named model tensor (measurement hook: lets a harness launch single
 * kernels of the kernel library on the resident weights).  NULL if unknown. */
void* pie_hip_driver_tensor_ptr(PieHipDriver* d, const char* name);

/*
 * Host-only planner hook (no GPU work): runs the forward-request planner and copies the
 * integer plan out so page-table arithmetic can be checked bit-exactly
 * (driver/portable/src/plan.hpp:36-45, plan.cpp:177-470).  out_i64 receives kv_slots[N];
 * out_i32 receives, back to back: positions[N], row_page_begin[N], row_kv_len[N], seq_len[R],
 * sample_rows[S], sample_indptr[R+1], then {R, N, S, max_kv_len, pure_decode, all_greedy,
 * has_user_masks}.  Returns the number of int32 values written, or -1 with the planner's
 * message in err.
 */
long long pie_hip_driver_plan(const PieForwardRequestDesc* f, int page_size, int total_pages,
                              long long* out_i64, int* out_i32, size_t out_i32_cap, char* err,
                              size_t err_cap);

#ifdef __cplusplus
}
#endif
#endif /* PIE_DRIVER_ABI_H */
