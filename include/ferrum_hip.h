/*
 * ferrum_hip.h -- C ABI of the MI355X (gfx950) backend for Ferrum's
 * quantized-matmul operators.
 *
 * Each entry point names the Ferrum interface it stands in for (paths are
 * relative to the Ferrum source tree).  A Rust `src/hip` backend would bind
 * these with `extern "C"` and implement the `MetalDevice` operator methods of
 * `src/ops` on top of them; GGUF super-blocks are uploaded verbatim.
 *
 * Conventions (the reference's, src/metal/mod.rs and src/ops/mod.rs):
 *   - every call returns fh_status; FH_OK is 0; nothing throws or aborts on
 *     bad input.  fh_last_error() returns a thread-local message for the most
 *     recent failure on the calling thread.
 *   - a device owns one HIP stream; operator calls enqueue on it and return.
 *     Results are readable after fh_synchronize() or through
 *     fh_buffer_download(), which waits for the stream first.
 *   - buffers and matrices belong to the device that created them; passing a
 *     foreign one fails with FH_ERR_DEVICE_MISMATCH.
 *   - a device and its objects are not thread-safe (Ferrum's handles are
 *     `Rc`, i.e. !Send + !Sync).
 *   - tensors are dense row-major; fh_view carries {buffer, byte offset,
 *     dtype}.  Activation and output views must be 16-byte aligned.
 *   - all element counts and indices must fit in 32 bits (src/ops/mod.rs:991).
 */
#ifndef FERRUM_HIP_H
#define FERRUM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int32_t fh_status;

/* Mirrors ferrum::Error (src/error.rs:3-51). */
enum {
    FH_OK = 0,
    FH_ERR_SHAPE = 1,
    FH_ERR_DTYPE = 2,
    FH_ERR_DEVICE_MISMATCH = 3,
    FH_ERR_RANGE = 4,
    FH_ERR_DISPATCH = 5,
    FH_ERR_SYNCHRONIZATION = 6,
    FH_ERR_ALLOCATION = 7,
    FH_ERR_GGUF = 8,
    FH_ERR_WEIGHT = 9,
    FH_ERR_PARAMETER = 10,
    FH_ERR_TOKEN = 11,
    FH_ERR_VALIDATION = 12
};

/* DType (src/tensor/mod.rs:5-11). */
enum { FH_F32 = 0, FH_F16 = 1, FH_BF16 = 2 };

/* GGML type ids of the supported formats (src/quantization.rs:24-49; IQ4_XS
 * and Q8_0 are the hybrid engine's Format::Iq4Xs and Format::Q8_0,
 * src/hybrid/weights.rs:29-60: 136-byte blocks of 256 weights and 34-byte
 * blocks of 32, src/loader/gguf.rs:91-121).  A row is a whole number of
 * blocks: a multiple of 256 weights, or of 32 for Q8_0 (src/hybrid/weights.rs:1167).
 * A Q8_0 matrix whose rows do not end on a run of eight blocks is kept on the
 * device with every row completed to such a run by empty blocks (scale and
 * quants zero; fh_qmatrix_device_ptr shows that layout, fh_qmatrix_byte_size and
 * fh_qmatrix_columns the caller's).  Every entry point that multiplies by such
 * a matrix first copies its activations to that width, zeros in the added
 * columns, into a block the device owns (one small launch; the block grows
 * outside recordings only), and then runs as on any other matrix (the added
 * terms are exact zeros).  fh_project_quantized_no_alloc has no room for
 * the copy and returns FH_ERR_SHAPE for such a matrix; fh_moe_ffn takes its
 * separate launches. */
enum { FH_GGML_Q8_0 = 8, FH_GGML_Q4_K = 12, FH_GGML_Q5_K = 13, FH_GGML_Q6_K = 14, FH_GGML_IQ4_XS = 23 };

typedef struct fh_device fh_device;
typedef struct fh_buffer fh_buffer;
typedef struct fh_qmatrix fh_qmatrix;
typedef struct fh_event fh_event;
typedef struct fh_graph fh_graph;

typedef struct fh_view {
    fh_buffer* buffer;
    size_t offset;  /* bytes */
    uint32_t dtype; /* FH_F32 / FH_F16 / FH_BF16 */
} fh_view;

typedef struct fh_device_props {
    char name[128];
    char arch[64];
    int32_t compute_units;
    int32_t wavefront;
    int32_t clock_khz;
    int32_t memory_clock_khz;
    int32_t memory_bus_bits;
    int32_t lds_bytes_per_block;
    uint64_t global_bytes;
    uint64_t l2_bytes;
} fh_device_props;

/* MoeRoutingPolicy (src/model/architecture.rs; consumed at src/ops/mod.rs:23-73). */
typedef struct fh_routing_policy {
    uint32_t experts;
    uint32_t top_k;
    uint32_t sigmoid;              /* 0 softmax over all experts, 1 sigmoid */
    uint32_t normalize_top_k_prob; /* divide by (sum of selected + epsilon) */
    float normalization_epsilon;
    float routed_scaling_factor;
} fh_routing_policy;

/* ---- device ---------------------------------------------------------------
 * MetalDevice::new / synchronize (src/metal/mod.rs:585-635).  Fails with
 * FH_ERR_DISPATCH when the GPU is not gfx950. */
fh_status fh_device_create(int32_t ordinal, fh_device** out);
void fh_device_destroy(fh_device* device);
fh_status fh_device_properties(const fh_device* device, fh_device_props* out);
fh_status fh_synchronize(fh_device* device);
const char* fh_last_error(void);
/* Kernel the most recent operator call selected: Output.metrics.operation
 * (src/ops/mod.rs:8-21), which the reference's tests assert on. */
const char* fh_last_operation(const fh_device* device);
/* Raw hipStream_t of the device, for interop and external event timing. */
void* fh_device_stream(fh_device* device);

/* Kernel-selection switches: the legacy::Tuning setters
 * (src/metal/legacy.rs:8-111), e.g. "k_quant_gemv_ksplit" with the same value
 * rule as set_k_quant_gemv_ksplit (0 or a power of two up to 8).  Unknown
 * keys or out-of-range values give FH_ERR_PARAMETER. */
fh_status fh_set_tuning(fh_device* device, const char* key, int64_t value);
fh_status fh_get_tuning(const fh_device* device, const char* key, int64_t* value);

/* ---- buffers ----------------------------------------------------------------
 * MetalDevice::allocate (zero-initialised, src/metal/mod.rs:727-734) and the
 * host copies behind Tensor::from_f32 / to_f32 (src/tensor/mod.rs). */
fh_status fh_buffer_alloc(fh_device* device, size_t bytes, fh_buffer** out);
void fh_buffer_free(fh_buffer* buffer);
size_t fh_buffer_size(const fh_buffer* buffer);
void* fh_buffer_device_ptr(fh_buffer* buffer);
fh_status fh_buffer_upload(fh_buffer* buffer, size_t offset, const void* src, size_t bytes);
fh_status fh_buffer_download(const fh_buffer* buffer, size_t offset, void* dst, size_t bytes);
fh_status fh_buffer_fill_zero(fh_buffer* buffer, size_t offset, size_t bytes);

/* ---- packed weights --------------------------------------------------------
 * QuantizedMatrix::from_reader (src/quantization.rs:86-111) together with
 * validate_gguf_quantized_payload (:212-261) and, for experts > 1,
 * QuantizedExpertMatrix::new (:147-165): a row-major [experts*rows, cols]
 * matrix of verbatim GGUF super-blocks.  `rows` is rows per expert.
 * Errors: FH_ERR_SHAPE (empty, cols % 256 or, for Q8_0, cols % 32; size overflow, length mismatch),
 * FH_ERR_GGUF (unsupported type, payload ends inside a block),
 * FH_ERR_WEIGHT (non-finite block scale). */
fh_status fh_qmatrix_create(fh_device* device, uint32_t ggml_type, uint64_t rows, uint64_t cols,
                            uint64_t experts, const void* packed, size_t packed_len,
                            fh_qmatrix** out);
void fh_qmatrix_destroy(fh_qmatrix* matrix);
uint64_t fh_qmatrix_rows(const fh_qmatrix* matrix);    /* rows per expert */
uint64_t fh_qmatrix_columns(const fh_qmatrix* matrix);
uint64_t fh_qmatrix_experts(const fh_qmatrix* matrix);
uint32_t fh_qmatrix_ggml_type(const fh_qmatrix* matrix);
size_t fh_qmatrix_byte_size(const fh_qmatrix* matrix);
void* fh_qmatrix_device_ptr(fh_qmatrix* matrix);

/* Whole-matrix dequantisation to [experts*rows, cols] in out.dtype.  The
 * reference has no host decoder for these formats; its per-element GPU
 * decoders q4_k_weight / q6_k_weight (src/metal/shaders/ops.metal:834-845,
 * 1316-1329) define the values.  f32 output is bit-exact. */
fh_status fh_dequantize(fh_device* device, const fh_qmatrix* weight, const fh_view* out);

/* MetalDevice::embedding_gather_quantized (src/ops/transformer.rs:299-360):
 * out[t, :] = dequantised row tokens[t], rounded to out.dtype.
 * FH_ERR_TOKEN when an id is >= rows. */
fh_status fh_embedding_gather_quantized(fh_device* device, const fh_qmatrix* weight,
                                        const uint32_t* tokens, size_t count, const fh_view* out);

/* ---- dense projection -------------------------------------------------------
 * MetalDevice::project_quantized (src/ops/transformer.rs:96-297):
 * Y[M,N] = X[M,K] * W[N,K]^T with f32 accumulation.  x is [m, K] in x.dtype,
 * y is [m, N] in y.dtype (the reference always uses y.dtype == x.dtype).
 * FH_ERR_SHAPE when m == 0, K exceeds u32::MAX - 32 or an index overflows;
 * FH_ERR_RANGE when a view is out of bounds, misaligned, or y overlaps x. */
fh_status fh_project_quantized(fh_device* device, const fh_qmatrix* weight, const fh_view* x,
                               uint32_t m, const fh_view* y);

/* fh_project_quantized for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Every row of x goes through the GEMV kernels (any m,
 * any dtype; same results as fh_project_quantized whenever that takes those kernels),
 * and the partial sums and row-tile counters a long-K launch needs live in a fixed 1 MiB
 * array inside the library, one copy per GPU, held until the process ends.  The call
 * makes no hipMalloc / hipFree and does not synchronise.  FH_ERR_SHAPE when a launch
 * would need more than 4096 counters (row tiles x m) or 1032192 bytes of partial sums
 * (K segments x m x N x 4), or for a Q8_0 matrix whose rows are stored padded (rows of
 * 32 n weights, n not a multiple of 8: the activations would need a widened copy); nothing
 * is launched then.  All calls on one GPU share the
 * array: calls that overlap in time on one GPU (two streams, two threads) race. */
fh_status fh_project_quantized_no_alloc(fh_device* device, const fh_qmatrix* weight,
                                        const fh_view* x, uint32_t m, const fh_view* y);

/* MetalDevice::argmax_rows (src/ops/transformer.rs:768-792, kernel
 * src/metal/shaders/ops.metal:2438-2464): greedy selection over the rows of a
 * logits matrix, the step after the lm_head projection.  out is an f32 carrier
 * [rows, 2] holding u32 bits: the first maximal index of the row and a flag
 * that is 1 when the row holds a non-finite value. */
fh_status fh_argmax_rows(fh_device* device, const fh_view* logits, uint32_t rows, uint32_t width,
                         const fh_view* out);

/* MetalDevice::add_rmsnorm (src/ops/mod.rs:762-820, kernel
 * src/metal/shaders/ops.metal:99-124) and the hybrid engine's h_add_rmsnorm
 * (src/hybrid/engine.rs:3322-3342, src/metal/shaders/hybrid.metal:1576-1595):
 * the residual add fused with the RMSNorm that feeds the next projection.
 * a, b, residual, normed are [rows, width], weight is [width], all of one
 * dtype.  residual = a + b rounded to that dtype (what a separate add
 * stores); normed = residual * rsqrt(mean(residual^2) + epsilon) * weight.
 * FH_ERR_SHAPE when the geometry is empty or the dtypes differ,
 * FH_ERR_PARAMETER unless epsilon is finite and positive, FH_ERR_RANGE when
 * an output overlaps an operand or the other output. */
fh_status fh_add_rmsnorm(fh_device* device, const fh_view* a, const fh_view* b, const fh_view* weight,
                         uint32_t rows, uint32_t width, float epsilon, const fh_view* residual,
                         const fh_view* normed);

/* ---- mixture of experts -----------------------------------------------------
 * MetalDevice::moe_route (src/ops/mod.rs:23-73; kernel ops.metal:1894-1957).
 * logits [tokens, experts]; bias (may be NULL) [experts] f32; metadata
 * [tokens*top_k, 3] f32 rows {expert id bits, token id bits, weight}, sorted
 * by expert id within a token. */
fh_status fh_moe_route(fh_device* device, const fh_view* logits, uint32_t tokens,
                       const fh_view* selection_bias, const fh_routing_policy* policy,
                       const fh_view* metadata);

/* MetalDevice::expert_assign (src/ops/mod.rs:75-115): out[a,:] =
 * hidden[token(a),:]; hidden [tokens, width], out [tokens*top_k, width]. */
fh_status fh_expert_assign(fh_device* device, const fh_view* hidden, uint32_t tokens,
                           uint32_t width, const fh_view* metadata, uint32_t top_k,
                           const fh_view* out);

/* MetalDevice::expert_project_quantized (src/ops/mod.rs:188-333, grouped and
 * tile forms :336-485): y[a, r] = sum_k x[a,k] * W[expert(a)*rows + r, k].
 * x [assignments, K], metadata [assignments, 3] f32, y [assignments, rows]. */
fh_status fh_expert_project_quantized(fh_device* device, const fh_qmatrix* weight,
                                      const fh_view* x, uint32_t assignments,
                                      const fh_view* metadata, const fh_view* y);

/* The hybrid engine's router and combine (f32 models; HybridModel::moe_ffn,
 * src/hybrid/engine.rs:2881-3092).
 *
 * fh_moe_route_ranked is h_moe_route (src/metal/shaders/hybrid.metal:2259-2319):
 * softmax over all experts or sigmoid, top-k with ties to the lower index,
 * weights divided by their sum when policy->normalize_top_k_prob is set, rows
 * kept in SELECTION order (rank 0 first) instead of expert-id order, and the
 * shared-expert gate sigmoid(dot(x[t], gate_vector)) written to shared_gate
 * [tokens] f32 (1 when gate_vector is NULL; nothing when shared_gate is NULL).
 * The hybrid engine's ids[] and weights[] are columns 0 and 2 of the metadata
 * rows; expert projections and combine take the rows as they are.  The
 * policy's epsilon and scaling apply as in fh_moe_route (the hybrid engine
 * uses 0 and 1); there is no selection bias.
 *
 * fh_expert_combine_shared is h_moe_combine (hybrid.metal:2374-2388):
 * out[t] = sum over ranks of w * down[row] + shared_gate[t] * shared[t]
 * (gate 1 when shared_gate is NULL), with fh_expert_combine's storage rounding
 * for 16-bit types. */
fh_status fh_moe_route_ranked(fh_device* device, const fh_view* logits, uint32_t tokens,
                              const fh_routing_policy* policy, const fh_view* x, const fh_view* gate_vector,
                              uint32_t hidden, const fh_view* metadata, const fh_view* shared_gate);
fh_status fh_expert_combine_shared(fh_device* device, const fh_view* in, const fh_view* metadata,
                                   uint32_t tokens, uint32_t hidden, uint32_t top_k, const fh_view* shared,
                                   const fh_view* shared_gate, const fh_view* out);

/* The hybrid engine's routed FFN in its own data layout: expert ids and route
 * weights are two [tokens, used] arrays (ids as u32 bits in an f32 carrier, as
 * the engine's Tensor::from_le_bytes(.., DType::F32, ..) holds them), not
 * metadata triples.  HybridModel::moe_ffn, src/hybrid/engine.rs:2881-3080.
 *
 * fh_hybrid_moe_route  = h_moe_route (src/metal/shaders/hybrid.metal:2259-2319):
 *   fh_moe_route_ranked writing ids, weights [tokens * top_k] and shared_gate.
 * fh_hybrid_project_id = HybridModel::project_id (engine.rs:3113-3148, kernels
 *   h_mv_id_*, hybrid.metal:2391-2425): route r multiplies activation row
 *   r / x_div of x [routes / x_div, K] by expert ids[r]; y is [routes, rows].
 *   An id that is not an expert gives a zero row.  FH_ERR_SHAPE when x_div
 *   does not divide routes.
 * fh_hybrid_moe_map    = h_moe_map (hybrid.metal:2321-2358): the expert-major
 *   order of routes, stable inside an expert: offsets [experts + 1], sorted
 *   [routes] (route at each row), position [routes] (row of each route).
 * fh_hybrid_moe_gather = h_moe_gather (hybrid.metal:2360-2370):
 *   out[p] = x[sorted[p] / used], x [routes / used, hidden].
 * fh_hybrid_project_mm_id = HybridModel::project_mm_id (engine.rs:3150-3220
 *   without arena slots, kernels h_mm_id_*): rows offsets[e] .. offsets[e+1]
 *   of x [routes, K] are multiplied by expert e; y [routes, rows] in the same
 *   row order.  The tiles are f16 (f32 rows are rounded first), as there.
 * fh_hybrid_moe_combine = h_moe_combine (hybrid.metal:2372-2388), f32:
 *   out[t] = sum_s weights[t, s] * down[row(t, s)] + shared_gate[t] * shared[t],
 *   row(t, s) = position[t * used + s], or the route itself when position is
 *   NULL (the engine's `identity`). */
fh_status fh_hybrid_moe_route(fh_device* device, const fh_view* logits, uint32_t tokens,
                              const fh_routing_policy* policy, const fh_view* x, const fh_view* gate_vector,
                              uint32_t hidden, const fh_view* ids, const fh_view* weights,
                              const fh_view* shared_gate);
/* HybridModel::project (src/hybrid/engine.rs:3407-3500) with its tiers
 * (MVB_MAX_ROWS = 4, MMS_MAX_ROWS = 32, :3584-3585): one row, or any row count
 * when `exact` is set (the engine's exact_math flag), multiplies exact f32
 * weights; 2..4 rows do the same row by row (the batched GEMV h_mvb_*); from 5
 * rows on f32 activations are rounded to f16 and take the tile kernels
 * (h_mms_* up to 32 rows, h_mm_* beyond), whatever gemm_f32_min_rows says.
 * fh_last_operation names the tier, e.g. "h_mms_q4_k". */
fh_status fh_hybrid_project(fh_device* device, const fh_qmatrix* weight, const fh_view* x, uint32_t m,
                            const fh_view* y, uint32_t exact);
fh_status fh_hybrid_project_id(fh_device* device, const fh_qmatrix* weight, const fh_view* x, const fh_view* ids,
                               uint32_t routes, uint32_t x_div, const fh_view* y);
/* fh_hybrid_project_id with the shared expert's projection in the same launch.
 * moe_ffn runs the shared expert as a dense FFN of three more per-row
 * projections right after routing (engine.rs:2925); in its identity branch
 * (a few routes) each is a launch of a few microseconds.  Here the shared
 * expert's `tokens` rows are further entries of the per-route kernel on the
 * dense matrix shared_weight (one expert's rows, columns and format): entry t
 * reads row t of shared_x [tokens, K] when that is given (the down projection:
 * the shared expert's own activated rows) and row t of x otherwise (gate and
 * up: x holds one row per token, tokens == routes / x_div), and writes row t
 * of shared_y [tokens, rows].  y and shared_y are bit for bit what
 * fh_hybrid_project_id and a one-row-at-a-time fh_hybrid_project write. */
fh_status fh_hybrid_project_id_with_shared(fh_device* device, const fh_qmatrix* weight,
                                           const fh_qmatrix* shared_weight, const fh_view* x, const fh_view* ids,
                                           uint32_t routes, uint32_t x_div, uint32_t tokens, const fh_view* shared_x,
                                           const fh_view* y, const fh_view* shared_y);
fh_status fh_hybrid_moe_map(fh_device* device, const fh_view* ids, uint32_t experts, uint32_t routes,
                            const fh_view* offsets, const fh_view* sorted, const fh_view* position);
fh_status fh_hybrid_moe_gather(fh_device* device, const fh_view* x, const fh_view* sorted, uint32_t hidden,
                               uint32_t used, uint32_t routes, const fh_view* out);
fh_status fh_hybrid_project_mm_id(fh_device* device, const fh_qmatrix* weight, const fh_view* x,
                                  const fh_view* offsets, uint32_t routes, const fh_view* y);
/* fh_hybrid_project_mm_id with the shared expert's projection in the same
 * launch: moe_ffn's prompt branch runs the shared expert's dense FFN
 * (engine.rs:2925) as three more tile GEMMs next to the three project_mm_id
 * calls.  Here row t of shared_x [tokens, K] is multiplied by the dense
 * shared_weight (one expert's rows, columns and format) into row t of
 * shared_y [tokens, rows] by the workgroups of the routed kernel, after their
 * own expert's rows; f32 rows are rounded to f16 like the routed ones.  Same
 * results as fh_hybrid_project_mm_id plus fh_hybrid_project to the matmul
 * tolerance; rows too wide for the kernel's LDS run as those two calls. */
fh_status fh_hybrid_project_mm_id_with_shared(fh_device* device, const fh_qmatrix* weight,
                                              const fh_qmatrix* shared_weight, const fh_view* x,
                                              const fh_view* offsets, uint32_t routes, uint32_t tokens,
                                              const fh_view* shared_x, const fh_view* y, const fh_view* shared_y);
fh_status fh_hybrid_moe_combine(fh_device* device, const fh_view* down, const fh_view* weights,
                                const fh_view* position, const fh_view* shared, const fh_view* shared_gate,
                                uint32_t hidden, uint32_t used, uint32_t tokens, const fh_view* out);

/* Input forms.  SparseMoe::forward (src/nn/moe.rs:222-390) encodes
 * expert_assign, the gate|up projection, expert_silu_mul and the down
 * projection back to back; with a handful of assignments each of them is a
 * launch that lasts microseconds.  These two entry points fold the copy or the
 * activation into the projection that follows and give the same bits as the
 * separate calls.  fh_expert_project_fused is good at every batch size for
 * 16-bit activations: beyond the per-assignment kernel the grouped kernel
 * gathers the token rows itself, and what it cannot read in place the library
 * stages in its scratch with the kernels of the separate calls.  With f32
 * activations (per-assignment kernel only) and in the dense
 * fh_project_silu_mul_quantized (per-row kernel only) the forms are for
 * decode-sized batches, and callers keep the separate calls beyond them.
 *
 * fh_expert_project_fused: input_form FH_INPUT_ROWS is
 * fh_expert_project_quantized; FH_INPUT_GATHER reads x as hidden [x_rows, K]
 * and row a uses hidden[token(a), :] (expert_assign, src/ops/mod.rs:75-115,
 * folded in); FH_INPUT_SILU_MUL reads x as [assignments, 2K], gate first, and
 * multiplies by round(round(silu(gate)) * up) in x's dtype (expert_silu_mul,
 * src/ops/mod.rs:487-508, folded in).
 * fh_project_silu_mul_quantized: the dense projection of FH_INPUT_SILU_MUL,
 * packed [m, 2K] -> y [m, N] (a shared expert's down projection). */
enum { FH_INPUT_ROWS = 0, FH_INPUT_GATHER = 1, FH_INPUT_SILU_MUL = 2 };
fh_status fh_expert_project_fused(fh_device* device, const fh_qmatrix* weight, const fh_view* x,
                                  uint32_t x_rows, uint32_t input_form, uint32_t assignments,
                                  const fh_view* metadata, const fh_view* y);
fh_status fh_project_silu_mul_quantized(fh_device* device, const fh_qmatrix* weight,
                                        const fh_view* packed, uint32_t m, const fh_view* y);

/* The routed projection with a shared expert in the same launch.  Models with
 * a shared expert run it as a dense FFN on every token next to the routed
 * experts (the hybrid engine's moe_ffn, src/hybrid/engine.rs:2925, right
 * after routing); in decode that is two more launches of a few microseconds.
 * Here the `tokens` rows of the shared expert are further batch entries of
 * fh_expert_project_fused's per-assignment kernel: y gets what
 * fh_expert_project_fused(weight, x, tokens, input_form, ..) writes and
 * shared_y [tokens, N] what fh_project_quantized(shared_weight, x) (gathered
 * form; shared_x must be NULL) or fh_project_silu_mul_quantized(shared_weight,
 * shared_x) (SiLU form; shared_x is the shared expert's own packed
 * [tokens, 2K] rows) writes, bit for bit while both would take that kernel.
 * shared_weight is dense with one expert's rows, columns and format;
 * input_form is FH_INPUT_GATHER or FH_INPUT_SILU_MUL.  Where
 * fh_expert_project_fused groups the assignments by expert (16-bit rows,
 * 32 assignments or more), the shared expert's tokens join the grouped
 * kernel as further groups of 16 or 32 tokens on the dense matrix (512
 * tokens: 41 us of dense tile GEMMs become +23 us in the two grouped
 * launches); results then agree with the separate calls to the matmul
 * tolerance, not bitwise.  Rows too wide for that kernel's LDS run as the
 * separate calls. */
fh_status fh_expert_project_with_shared(fh_device* device, const fh_qmatrix* weight,
                                        const fh_qmatrix* shared_weight, const fh_view* x, uint32_t tokens,
                                        uint32_t input_form, uint32_t assignments, const fh_view* metadata,
                                        const fh_view* shared_x, const fh_view* y, const fh_view* shared_y);

/* MetalDevice::expert_silu_mul (src/ops/mod.rs:487-508): in [A, 2*I] (gate
 * first), out [A, I] = round(silu(gate)) * up, stored in out.dtype. */
fh_status fh_expert_silu_mul(fh_device* device, const fh_view* in, uint32_t assignments,
                             uint32_t intermediate, const fh_view* out);

/* MetalDevice::expert_combine (src/ops/mod.rs:510-551): out[t,c] = sum over
 * the token's top_k rows, in metadata order, of round(round(w) * v). */
fh_status fh_expert_combine(fh_device* device, const fh_view* in, const fh_view* metadata,
                            uint32_t tokens, uint32_t hidden, uint32_t top_k, const fh_view* out);

/* SparseMoe::forward (src/nn/moe.rs:222-390) in one call: route, gate|up projection, SiLU*up,
 * down projection and weighted combine of `tokens` rows, with the hybrid engine's shared expert
 * (HybridModel::moe_ffn, src/hybrid/engine.rs:2881-3092) when shared_input [2*I_s, H] (gate rows
 * first) and shared_output [H, I_s] are given; shared_gate (may be NULL) [tokens] f32 scales its
 * rows.  hidden [tokens, H], router_logits [tokens, experts] (the router's own dense layer is the
 * caller's), selection_bias as in fh_moe_route, out [tokens, H] in the activation dtype.  The
 * steps are exactly those the calls above would make one by one, with expert_assign and
 * expert_silu_mul folded into the projections and the shared expert riding in the routed launches
 * where fh_expert_project_with_shared allows, so the result has their bits (a single token's
 * weighted sum is added inside the down projection's launch, and its routing inside the gate|up
 * launch: the same arithmetic in two launches; many tokens' records are grouped by expert once for
 * both projections).  Tokens are taken in
 * chunks whose routing temporaries stay under the tuning value moe_routing_temporary_limit
 * (src/nn/moe.rs:232-256); the temporaries live in a workspace the library keeps per device,
 * which grows outside recordings only (run the call once before recording it). */
fh_status fh_moe_ffn(fh_device* device, const fh_view* hidden, const fh_view* router_logits, uint32_t tokens,
                     const fh_view* selection_bias, const fh_routing_policy* policy,
                     const fh_qmatrix* input_experts, const fh_qmatrix* output_experts,
                     const fh_qmatrix* shared_input, const fh_qmatrix* shared_output,
                     const fh_view* shared_gate, const fh_view* out);

/* ---- batched execution ---------------------------------------------------------
 * MetalDevice::execution_with_shared_encoder / Execution::finish
 * (src/metal/mod.rs:263-278, 563-572): operator calls between begin and end
 * are recorded instead of run (up to the reference's batch of 1,024
 * dispatches and beyond) and replayed as one HIP graph by fh_graph_launch.
 * While recording, calls that must wait for the GPU or allocate (buffer and
 * matrix creation, upload, download, embedding gather) fail with
 * FH_ERR_SYNCHRONIZATION; size the outputs before.  A nested begin is an
 * error, like a nested execution. */
fh_status fh_execution_begin(fh_device* device);
fh_status fh_execution_end(fh_device* device, fh_graph** out);
fh_status fh_graph_launch(fh_graph* graph);
void fh_graph_destroy(fh_graph* graph);

/* ---- timing ------------------------------------------------------------------
 * Events on the device's own stream, for the per-dispatch GPU time the
 * reference reads from its command buffers (src/metal/mod.rs:601-604). */
fh_status fh_event_create(fh_device* device, fh_event** out);
void fh_event_destroy(fh_event* event);
fh_status fh_event_record(fh_event* event);
fh_status fh_event_elapsed_ms(fh_event* start, fh_event* stop, float* ms);

#ifdef __cplusplus
}
#endif
#endif /* FERRUM_HIP_H */
