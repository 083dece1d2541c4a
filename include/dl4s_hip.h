/*
 * dl4s_hip.h -- C ABI of libdl4s_hip.so: an MI355X (gfx950) backend for the attention
 * forward path of DL4S (ScaledDotProductAttention / MultiHeadAttention and the engine
 * primitives those layers call), fp32, one GPU.
 *
 * The library owns the device context, one HIP stream, a pooled allocator and every kernel
 * launch.  Handles are raw device pointers; an offset view is plain pointer arithmetic and is
 * never passed to dl4s_hip_free.  Every function is callable from any thread, returns 0 on
 * success or a negative dl4s_hip_status, never aborts and never throws across the ABI; the
 * message for the last failure on the calling thread is dl4s_hip_last_error().
 *
 * Compute entry points only ENQUEUE work on the context's stream.  Results are visible to a
 * following dl4s_hip_assign_d2h / dl4s_hip_get_value (which wait for the stream) or after
 * dl4s_hip_sync.  Host pointers handed to dl4s_hip_assign_h2d may be reused as soon as the
 * call returns.
 *
 * Citations are to the reference sources, relative to Sources/DL4S/.
 */
#ifndef DL4S_HIP_H
#define DL4S_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dl4s_hip_ctx dl4s_hip_ctx;

typedef enum dl4s_hip_status {
    DL4S_HIP_OK = 0,
    DL4S_HIP_EINVALID_ARG = -1, /* null pointer, negative size, unknown enum value */
    DL4S_HIP_ESHAPE = -2,       /* operand shapes do not fit each other (the reference traps with precondition) */
    DL4S_HIP_EOOM = -3,         /* device allocation failed */
    DL4S_HIP_EHIP = -4,         /* a HIP runtime call failed; the message holds hipGetErrorString */
    DL4S_HIP_EUNSUPPORTED = -5  /* valid request outside what this backend implements */
} dl4s_hip_status;

#define DL4S_HIP_MAX_DIM 8

/* ------------------------------------------------------------------ context / device */
/* Engine/Engine.swift:30-35 (DeviceType): one context stands for the `HIP` device type. */
int dl4s_hip_create(int device_ordinal, dl4s_hip_ctx **out_ctx);
int dl4s_hip_destroy(dl4s_hip_ctx *ctx);
const char *dl4s_hip_last_error(void);
int dl4s_hip_sync(dl4s_hip_ctx *ctx);
/* Number of compute units and device name (for roofline reports). */
int dl4s_hip_device_info(dl4s_hip_ctx *ctx, int *out_cu_count, int *out_clock_khz, char *name_buf, size_t name_len);
/* Stream-ordered timer on the context's stream (HIP events): begin, enqueue work, end.
 * dl4s_hip_timer_end waits for the stop event and returns the elapsed milliseconds. */
int dl4s_hip_timer_begin(dl4s_hip_ctx *ctx);
int dl4s_hip_timer_end(dl4s_hip_ctx *ctx, float *out_ms);

/* ------------------------------------------------------------------ recorded call sequences (HIP graphs)
 * No counterpart in the reference.  A fixed sequence of calls on fixed buffers (one layer, one decode step at a fixed
 * length) costs about 3 us of launch latency per kernel when it is issued call by call and about 1.8 us when it is
 * replayed from a graph.  Between dl4s_hip_graph_begin and dl4s_hip_graph_end the calls on this context are recorded
 * instead of run; dl4s_hip_graph_launch replays them, in stream order with everything else on the context.
 *
 * What can be recorded: every entry point that only enqueues kernels or device-to-device copies.  Entry points that
 * wait for the stream, copy to or from host memory (dl4s_hip_sync, the timer, dl4s_hip_assign_h2d / _d2h, the single
 * value getters and setters, dl4s_hip_argmax_f32) or that would have to allocate (dl4s_hip_alloc without a pooled
 * block of that size, a call that needs more library scratch than is there) return DL4S_HIP_EUNSUPPORTED and leave the
 * recording open.  Run the same calls once before recording them: that sizes the scratch block.
 *
 * A graph holds the addresses it was recorded with.  Every buffer that the recorded calls read or write must stay
 * allocated for as long as the graph is replayed; inputs are read at replay time, so new data in the same buffers gives
 * new results.  Temporaries may be allocated and freed inside the recording as usual: a block handed to dl4s_hip_free
 * while recording stays reserved for the graph and returns to the pool when the graph is destroyed.
 * Some calls use the library's scratch block: if a later call regrows it, dl4s_hip_graph_launch refuses the graph
 * (DL4S_HIP_EUNSUPPORTED) and it has to be recorded again.  One recording at a time per context, made and replayed
 * from one host thread at a time.
 *
 * Graphs cannot be replayed under rocprofv3: its queue interception rejects the packets of a graph launch
 * (HSA_STATUS_ERROR_INVALID_PACKET_FORMAT, ROCm 7.2) and the queue is aborted.  dl4s_hip_graph_supported returns 0 when
 * the process was started by rocprofv3, and dl4s_hip_graph_begin then refuses with DL4S_HIP_EUNSUPPORTED.
 *
 * dl4s_hip_graph_end with out_graph == NULL gives the recording up, and so does dl4s_hip_destroy.  Destroy a context's
 * graphs before the context. */
typedef struct dl4s_hip_graph dl4s_hip_graph;
int dl4s_hip_graph_supported(void);
int dl4s_hip_graph_begin(dl4s_hip_ctx *ctx);
int dl4s_hip_graph_end(dl4s_hip_ctx *ctx, dl4s_hip_graph **out_graph);
int dl4s_hip_graph_launch(dl4s_hip_ctx *ctx, dl4s_hip_graph *graph);
int dl4s_hip_graph_node_count(dl4s_hip_ctx *ctx, const dl4s_hip_graph *graph, size_t *out_nodes);
int dl4s_hip_graph_destroy(dl4s_hip_ctx *ctx, dl4s_hip_graph *graph);

/* ------------------------------------------------------- MemoryOperatorsType subset */
/* Engine/Engine.swift:49,55 allocateBuffer.  Memory is NOT zeroed (the reference's is not either,
 * Engine/CPU/CPU.swift:71-96).  bytes == 0 yields a valid unique pointer. */
int dl4s_hip_alloc(dl4s_hip_ctx *ctx, size_t bytes, void **out_ptr);
/* Engine/Engine.swift:59,63 free.  Stream-ordered: the block returns to the pool and may be
 * handed out again at once, because every consumer runs on the one stream
 * (Tensor/Tensor.swift:38-42 frees from deinit right after the last use was enqueued). */
int dl4s_hip_free(dl4s_hip_ctx *ctx, void *ptr);
/* Engine/Engine.swift:70 assign(from: UnsafeBufferPointer, to: Buffer) -- host to device. */
int dl4s_hip_assign_h2d(dl4s_hip_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
/* Engine/Engine.swift:77 assign(from: Buffer, to: Buffer) -- device to device. */
int dl4s_hip_assign_d2d(dl4s_hip_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes);
/* Engine/Engine.swift:84 assign(from: Buffer, to: UnsafeMutableBufferPointer) -- device to host; waits. */
int dl4s_hip_assign_d2h(dl4s_hip_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);
/* Engine/Engine.swift:88 getValue / :132 setPointee, for Float. */
int dl4s_hip_get_value_f32(dl4s_hip_ctx *ctx, const float *src_dev, float *out_value);
int dl4s_hip_set_pointee_f32(dl4s_hip_ctx *ctx, float *dst_dev, float value);
/* Engine/Engine.swift:92 getSize: bytes from ptr to the end of its allocation (works for offset views). */
int dl4s_hip_get_size(dl4s_hip_ctx *ctx, const void *ptr, size_t *out_bytes);
/* Bytes currently handed out / held by the pool (leak checks; Engine/CPU/CPU.swift:38-44 traces the same). */
int dl4s_hip_mem_stats(dl4s_hip_ctx *ctx, size_t *out_bytes_in_use, size_t *out_bytes_pooled);
/* Returns pooled blocks to the driver, largest first, until at most keep_bytes stay pooled (0: all of them).  The pool
 * keeps every freed block for the next allocation of its size and otherwise lets go only when an allocation fails; a
 * caller that is done with a phase of large temporaries (the attention gradients take B*H*Lq*Lk floats) gives the
 * memory back with this.  Waits for the stream (a pooled block may still be in use by work in flight); refused while
 * a call sequence is being recorded.  No counterpart in the reference, whose buffers go back to malloc one by one. */
int dl4s_hip_pool_trim(dl4s_hip_ctx *ctx, size_t keep_bytes);

/* ------------------------------------------------------------ fused attention entry */
/* Mask descriptor.  The reference takes a dense float tensor (1 = blocked, 0 = keep, any value is
 * a scaled penalty) broadcastable to [B,H,Lq,Lk] and computes  scores - mask * 1e9
 * (NN/Models/Transformer/ScaledDotProductAttention.swift:55-57).  DENSE_F32 is that tensor;
 * the structured kinds describe the masks TransformerUtil.swift:29-50 builds without
 * materialising them and give bit-identical results to DENSE_F32 on the same logical mask. */
typedef enum dl4s_mask_kind {
    DL4S_MASK_NONE = 0,
    DL4S_MASK_DENSE_F32 = 1,             /* dense: device ptr + shape[4], a 1 in shape = broadcast axis */
    DL4S_MASK_CAUSAL = 2,                /* blocked where key j > query i (bandMatrix(below:-1, above:nil)) */
    DL4S_MASK_KEY_LENGTHS = 3,           /* blocked where key j >= lengths[b] (makeEncoderMasks) */
    DL4S_MASK_CAUSAL_OR_KEY_LENGTHS = 4  /* union of the two (makeDecoderMasks) */
} dl4s_mask_kind;

typedef struct dl4s_mask_desc {
    int32_t kind;            /* dl4s_mask_kind */
    const float *dense;      /* DENSE_F32: device pointer, row-major, shape below */
    int64_t shape[4];        /* DENSE_F32: right-aligned to [B,H,Lq,Lk]; each entry is 1 or the full size */
    const int32_t *lengths;  /* KEY_LENGTHS kinds: device pointer to B valid lengths */
    const uint8_t *classes;  /* DENSE_F32, optional: the mask's tile classes as dl4s_hip_mask_classify_f32 left them for
                                this mask tensor and these extents; NULL = the attention call classifies the mask itself */
} dl4s_mask_desc;

/* Every layer of a model receives the same mask tensor (TransformerEncoder.swift:63, TransformerDecoder.swift:53-54 build
 * it once per forward pass), and an attention call under a dense mask first sorts the mask's 32 x 32 tiles into all
 * zeros / all ones / mixed (one small launch, about 5 us).  A caller can do that once per mask instead:
 *   dl4s_hip_mask_classes_size      bytes of device memory the classes of this mask take (host arithmetic only)
 *   dl4s_hip_mask_classify_f32      writes them to `classes` (device memory of that size, the caller's)
 * and passes the pointer in dl4s_mask_desc.classes of every attention call (forward, forward with statistics,
 * gradients) on the same mask tensor, B, H, Lq and Lk.  The classes describe the mask's values: classify again after
 * writing into the mask.  Results are the bits of the call that classifies by itself.  No counterpart in the reference. */
/* The masks the reference's builders make are structured: makeEncoderMasks blocks the keys from a sequence's length on,
 * makeDecoderMasks adds the keys after the query (TransformerUtil.swift:29-50), and the layers receive them as dense
 * tensors.  dl4s_hip_mask_describe_f32 looks at a dense mask once and, when its values are exactly those of
 * DL4S_MASK_NONE (all zeros), DL4S_MASK_KEY_LENGTHS, DL4S_MASK_CAUSAL or DL4S_MASK_CAUSAL_OR_KEY_LENGTHS, writes that
 * descriptor to *out, with the valid key counts in `lengths` (device int32 [B], the caller's; it must stay allocated
 * while *out is used); any other mask comes back as the dense descriptor it was.  An attention call gives the same bits
 * under either descriptor, and the structured one reads no mask values.  The call waits for the context's stream and
 * reads B + 1 integers back, so it is meant to run once per mask tensor (not inside a recorded sequence); describe
 * again after writing into the mask.  A mask with a head axis, or a query axis without a key axis, is not looked at.
 * No counterpart in the reference. */
int dl4s_hip_mask_describe_f32(dl4s_hip_ctx *ctx, const dl4s_mask_desc *mask, int64_t B, int64_t H, int64_t Lq, int64_t Lk,
                               int32_t *lengths, dl4s_mask_desc *out);
int dl4s_hip_mask_classes_size(const dl4s_mask_desc *mask, int64_t B, int64_t H, int64_t Lq, int64_t Lk, size_t *out_bytes);
int dl4s_hip_mask_classify_f32(dl4s_hip_ctx *ctx, const dl4s_mask_desc *mask, int64_t B, int64_t H, int64_t Lq, int64_t Lk,
                               uint8_t *classes);

/* flags for dl4s_hip_sdpa_fwd_f32 */
#define DL4S_SDPA_STRICT 1u /* visit every key tile even where the mask blocks all of it.  Without it fully blocked
                               tiles are skipped - those a structured mask describes, and the all-ones 32 x 32 tiles
                               of a dense mask in query blocks whose every row keeps an unblocked key (a zero) - which
                               is exact as long as K and V hold finite values at blocked positions (the reference
                               computes 0 * v there, so a NaN/Inf in V or K at a blocked key reaches the output only
                               in strict mode).  Fully blocked rows are never skipped: they come out as the reference computes
                               them - uniform while their scores stay within +-32, shared by the keys of the highest
                               bucket of fl(s - 1e9) on the grid of 64 that floats have next to 1e9 beyond that. */
#define DL4S_SDPA_TOKEN_MAJOR 2u /* q, out are [B,Lq,H,d] and k, v are [B,Lk,H,d] (the layout the projections of
                                    MultiHeadAttention produce, NN/Models/Transformer/MultiHeadAttention.swift:105-107
                                    before its permutes :109-111, and the layout its output permute :117 produces), so a
                                    caller can drop the four permuteAxes copies.  Needs the MFMA kernel's conditions (see
                                    dl4s_hip_sdpa_fwd_f32). */
#define DL4S_SDPA_NO_KEY_SPLIT 4u /* small launches (fewer 32-query blocks than about two per SIMD) normally split each
                                     block's keys over the 4 wavefronts of a workgroup (head dims up to 64) or over
                                     several workgroups (head dims above 64) and merge the partial softmax results;
                                     this flag keeps the unsplit kernel.  The two agree within rounding (different
                                     summation order over keys), each well inside the parity tolerance. */

/* out = softmax((q * inv_temperature) . k^T - mask * 1e9, axis = keys) . v
 * NN/Models/Transformer/ScaledDotProductAttention.swift:43-64.  q [B,H,Lq,dk], k [B,H,Lk,dk],
 * v [B,H,Lk,dv], out [B,H,Lq,dv], all row-major contiguous device fp32.  inv_temperature is the
 * fp32 reciprocal the reference forms once (Engine/CPU/CPUEngine.swift:635).  mask may be NULL
 * (= DL4S_MASK_NONE).  dk = dv, a multiple of 4 and at most 128, with 16-byte aligned tensors runs
 * a fused MFMA kernel written for tiles of 16, 32, 48, 64, 80, 96 or 128 columns; a head dim between two
 * widths is padded with zero columns on the fly and costs what the wider tile costs.  Even head dims
 * from 66 to 94 that are not a multiple of 4 run the 96-wide kernel as they are (8-byte aligned
 * tensors, launches that fill the GPU).  dk = dv above 128 up to 256 (a multiple of 4, aligned) runs
 * the same scheme on tiles of 160, 192 or 256 columns.  Other head dims up to 256 (dk != dv, odd,
 * unaligned tensors) run the same kernels on zero-padded copies of the operands, which the call
 * allocates from the context's pool, when the problem is large enough to pay for the copies; small
 * problems of such head dims run a plain fused kernel.  Head dims above 256 are refused. */
int dl4s_hip_sdpa_fwd_f32(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out,
                          int64_t B, int64_t H, int64_t Lq, int64_t Lk, int64_t dk, int64_t dv,
                          float inv_temperature, const dl4s_mask_desc *mask, uint32_t flags);

/* Training form of the fused attention (key dim = value dim = d; MFMA kernels for d a multiple of 4 up to 256 and 16-byte
 * aligned tensors - above 128 the gradients are batched MFMA products around one elementwise pass that forms its own row
 * statistics (stats is not read there), head-major layout only -
 * plain kernels for what those do not take, up to 256).  The reference differentiates ScaledDotProductAttention through
 * the backward closures of its primitive operators (Tensor/Operators/Matrix.swift:139-174 for the products through the
 * subscript views and the stack of broadcastMatrixMultiplied :79-117, Binary.swift:235-300 for e / sum,
 * Reduce.swift:35-62, Unary.swift:33-55 for exp, Binary.swift:161-224 for the subtractions); a backend that fuses the
 * forward pass has to supply the gradient itself, attached as the TensorContext of the hook's result:
 *   dl4s_hip_sdpa_fwd_stats_f32  the forward pass, also leaving two statistics per row in stats [B,H,Lq,2]
 *                                (the maximum the weights were formed against and the reciprocal of their sum;
 *                                opaque to the caller)
 *   dl4s_hip_sdpa_bwd_f32        dq, dk, dv for the upstream gradient dout of out, from q, k, v, out, stats and the
 *                                same mask and flags as the forward call (the mask takes no gradient)
 * Layouts follow the forward call ([B,H,L,d], or [B,L,H,d] with DL4S_SDPA_TOKEN_MAJOR; stats is always [B,H,Lq,2]).
 * The gradient call takes the route the forward call took (MFMA kernels for d a multiple of 4 up to 256 with 16-byte
 * aligned q, k, v, out; the same kernels on zero-padded copies for other d up to 256 on large problems; the plain
 * kernels otherwise) because the two kinds of kernels keep the statistics in different forms: pass both calls the same
 * tensors and extents.  On the direct MFMA route dout, dq, dk, dv must be 16-byte aligned too (DL4S_HIP_EUNSUPPORTED
 * otherwise).
 * Large launches form the scores once: the dK/dV kernel stores its dS tiles in a scratch tensor of B*H*Lk*Lq floats
 * from the context's pool and a second kernel contracts them with K.  The scratch is bounded by 24 GiB or by the
 * environment variable DL4S_HIP_BWD_SCRATCH_MAX_BYTES (0 = never); beyond the bound, or when the pool cannot supply it,
 * two self-contained kernels run that form the scores twice.
 * Deterministic: no atomics, the same bits on every run. */
int dl4s_hip_sdpa_fwd_stats_f32(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, float *out, float *stats,
                                int64_t B, int64_t H, int64_t Lq, int64_t Lk, int64_t d, float inv_temperature,
                                const dl4s_mask_desc *mask, uint32_t flags);
int dl4s_hip_sdpa_bwd_f32(dl4s_hip_ctx *ctx, const float *q, const float *k, const float *v, const float *out,
                          const float *stats, const float *dout, float *dq, float *dk, float *dv, int64_t B, int64_t H,
                          int64_t Lq, int64_t Lk, int64_t d, float inv_temperature, const dl4s_mask_desc *mask, uint32_t flags);

/* One decode step: the same attention with Lq = 1 over the first T rows of a key/value cache laid
 * out [B,H,Tcap,d] (d from 1 to 256; the kernel is instantiated for rows of 32, 64, 96, 128 and 256 floats and other
 * head dims run the next wider one with idle lanes; with d a multiple of 4 and q, the caches and the new rows 16-byte
 * aligned a lane reads its piece of a row with one 128-bit load, otherwise with 64-bit loads (d even, 8-byte aligned) or one
 * float at a time).  q, out [B,H,1,d].  The reference has no cache (greedy decoding re-runs
 * the prefix, NN/Models/Transformer/Transformer.swift:118-137); the result equals its
 * ScaledDotProductAttention on the gathered [B,H,T,d] tensors, no mask. */
int dl4s_hip_sdpa_decode_f32(dl4s_hip_ctx *ctx, const float *q, const float *kcache, const float *vcache,
                             float *out, int64_t B, int64_t H, int64_t T, int64_t Tcap, int64_t d,
                             float inv_temperature);
/* The same with a valid key count per batch element (device int32 lengths[B]): what ScaledDotProductAttention gives on the
 * gathered [B,H,T,d] tensors under the mask of makeEncoderMasks, m[b,0,0,j] = (j >= lengths[b])
 * (NN/Models/Transformer/TransformerUtil.swift:29-36).  With 1 <= lengths[b] the blocked keys have weight exactly zero in
 * the reference and are not visited here (exact while K and V are finite there, as for the prefill kernels without
 * DL4S_SDPA_STRICT); lengths[b] <= 0 blocks every key and the row comes out over all T keys (uniform for scores within +-32), as in the
 * reference; lengths[b] >= T blocks nothing.  lengths == NULL is dl4s_hip_sdpa_decode_f32. */
int dl4s_hip_sdpa_decode_lengths_f32(dl4s_hip_ctx *ctx, const float *q, const float *kcache, const float *vcache,
                                     float *out, int64_t B, int64_t H, int64_t T, int64_t Tcap, int64_t d,
                                     float inv_temperature, const int32_t *lengths);
/* dl4s_hip_sdpa_decode_f32 for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments, same kernels, same bits;
 * the partial records of a decode that is split over the keys live in a fixed 4 MiB block of the library's own device
 * memory (one per GPU, held until the process ends) instead of the context's growable scratch block, and the call
 * makes no allocating or freeing runtime call.  A problem whose records do not fit - B*H pairs times the number of key
 * splits times (the row width the kernel runs at + 4) floats above 4 MiB - is refused with DL4S_HIP_EUNSUPPORTED; the split rule aims at 16 wavefronts
 * per compute unit, so on a 256-CU GPU it asks for about 2048 records (2.1 MiB at d = 256) at most and the limit guards
 * larger GPUs.  Every call on a GPU shares that GPU's block: calls on one context are ordered by its stream, and a call
 * on another context of the same GPU first makes its stream wait for the last user's (an event created with the
 * context).  What stays the caller's job: replays of a recorded graph that holds this call are outside that
 * bookkeeping and race with calls on other contexts that overlap them in time.  Nothing in the block has to start at
 * zero (every record a call reads was written by that call). */
int dl4s_hip_sdpa_decode_noalloc_f32(dl4s_hip_ctx *ctx, const float *q, const float *kcache, const float *vcache,
                                     float *out, int64_t B, int64_t H, int64_t T, int64_t Tcap, int64_t d,
                                     float inv_temperature);
/* Writes k_new, v_new [B,H,1,d] into row `pos` of the caches [B,H,Tcap,d]
 * (replaces the concatenation a cache-less caller would do with Engine.stack). */
int dl4s_hip_kv_append_f32(dl4s_hip_ctx *ctx, float *kcache, float *vcache, const float *k_new,
                           const float *v_new, int64_t B, int64_t H, int64_t pos, int64_t Tcap, int64_t d);
/* Append at row `pos`, then attend over rows 0..pos (T = pos + 1) in one call. */
int dl4s_hip_sdpa_decode_step_f32(dl4s_hip_ctx *ctx, const float *q, float *kcache, float *vcache,
                                  const float *k_new, const float *v_new, float *out, int64_t B, int64_t H,
                                  int64_t pos, int64_t Tcap, int64_t d, float inv_temperature);
/* ---- a decoding step whose token and position live in device memory (no counterpart in the reference).
 * A step of cached decoding has the same shapes at every position; with the position and the chosen token kept in device
 * memory the calls of one step can be recorded once (dl4s_hip_graph_begin) and replayed for every later position.
 *   dl4s_hip_embed_at_f32            result[D] = table[*token_dev] * (*scale) + positions[*position_dev]; a token outside
 *                                    [0, vocab) embeds as zeros, a position outside [0, position_rows) adds nothing
 *   dl4s_hip_sdpa_decode_step_at_f32 dl4s_hip_sdpa_decode_step_f32 with pos = *pos_dev (one workgroup per (batch, head)
 *                                    pair, no key split); a value outside [0, Tcap) leaves caches and output untouched
 *   dl4s_hip_argmax_to_f32           index of the first maximum of values[0..count) written to *out_index_dev (what
 *                                    dl4s_hip_argmax_f32 returns), then *counter_dev += 1 when counter_dev != NULL
 * scale is a host pointer (or NULL), read when the call is made. */
int dl4s_hip_embed_at_f32(dl4s_hip_ctx *ctx, const float *table, int64_t vocab, int64_t D, const int32_t *token_dev,
                          const float *scale, const float *positions, int64_t position_rows, const int32_t *position_dev,
                          float *result);
int dl4s_hip_sdpa_decode_step_at_f32(dl4s_hip_ctx *ctx, const float *q, float *kcache, float *vcache, const float *k_new,
                                     const float *v_new, float *out, int64_t B, int64_t H, const int32_t *pos_dev,
                                     int64_t Tcap, int64_t d, float inv_temperature);
int dl4s_hip_argmax_to_f32(dl4s_hip_ctx *ctx, const float *values, int64_t count, int32_t *out_index_dev,
                           int32_t *counter_dev);

/* ------------------------------------------------------------------ EngineType subset */
/* The primitives the layers on the path call (Engine/Engine.swift:143-581); fp32 only.
 * `result` may alias an input wherever the reference allows it (same-shape elementwise ops). */
int dl4s_hip_fill_f32(dl4s_hip_ctx *ctx, float value, float *result, int64_t count);                     /* :153 */
int dl4s_hip_vadd_f32(dl4s_hip_ctx *ctx, const float *lhs, const float *rhs, float *result, int64_t count); /* :161 */
int dl4s_hip_vneg_f32(dl4s_hip_ctx *ctx, const float *val, float *result, int64_t count);                /* :168 */
int dl4s_hip_vsub_f32(dl4s_hip_ctx *ctx, const float *lhs, const float *rhs, float *result, int64_t count); /* :176 */
int dl4s_hip_vmul_f32(dl4s_hip_ctx *ctx, const float *lhs, const float *rhs, float *result, int64_t count); /* :184 */
int dl4s_hip_vdiv_f32(dl4s_hip_ctx *ctx, const float *lhs, const float *rhs, float *result, int64_t count); /* :192 */
/* :225 gemm: row-major result[M,N] = alpha * op(lhs) . op(rhs) + beta * result; shapes are the STORED
 * shapes of lhs and rhs.  beta != 0 really accumulates (cblas semantics of the MKL/Accelerate builds,
 * Engine/CPU/Numeric/CPUFloat.swift:268-279). */
int dl4s_hip_gemm_f32(dl4s_hip_ctx *ctx, const float *lhs, int64_t lhs_rows, int64_t lhs_cols,
                      const float *rhs, int64_t rhs_rows, int64_t rhs_cols, float *result,
                      float alpha, float beta, int transpose_first, int transpose_second);
/* Strided-batched form of the same gemm: `batch` problems, element strides between consecutive
 * operands (0 = shared).  One launch replaces the per-slice loop + stack of
 * Tensor/Operators/Matrix.swift:106-116. */
int dl4s_hip_gemm_batched_f32(dl4s_hip_ctx *ctx, const float *lhs, int64_t lhs_rows, int64_t lhs_cols,
                              int64_t lhs_stride, const float *rhs, int64_t rhs_rows, int64_t rhs_cols,
                              int64_t rhs_stride, float *result, int64_t result_stride, int64_t batch,
                              float alpha, float beta, int transpose_first, int transpose_second);
/* Grouped form: `count` (at most 4) products of one shape whose operands lie anywhere (host arrays of
 * device pointers; entries may repeat), in one launch - the three projections of
 * NN/Models/Transformer/MultiHeadAttention.swift:105-107, which the reference issues as three
 * broadcastMatrixMultiplied calls.  Every product gets the bits the single call gives. */
int dl4s_hip_gemm_grouped_f32(dl4s_hip_ctx *ctx, int count, const float *const *lhs, int64_t lhs_rows, int64_t lhs_cols,
                              const float *const *rhs, int64_t rhs_rows, int64_t rhs_cols, float *const *result,
                              float alpha, float beta, int transpose_first, int transpose_second);
/* :233 band: copies columns max(0,i-below) .. min(cols,i+above+1)-1 of each row i; other elements of
 * result are left untouched (the caller zero-fills first, Tensor/Operators/UtilOps.swift:117-121).
 * has_below / has_above == 0 stand for nil. */
int dl4s_hip_band_f32(dl4s_hip_ctx *ctx, const float *buffer, float *result, int64_t rows, int64_t cols,
                      int has_below, int64_t below, int has_above, int64_t above);
/* :242-263 broadcastAdd/Sub/Mul/Div.  Shapes right-aligned, size-1 axes broadcast.  Sub and Div use
 * the reference's scalar forms where it does (x + (-s), x * (1/s); Engine/CPU/CPUEngine.swift:601-637). */
typedef enum dl4s_binary_op { DL4S_OP_ADD = 0, DL4S_OP_SUB = 1, DL4S_OP_MUL = 2, DL4S_OP_DIV = 3 } dl4s_binary_op;
int dl4s_hip_broadcast_f32(dl4s_hip_ctx *ctx, int op, const float *lhs, const int64_t *lhs_shape, int lhs_dim,
                           const float *rhs, const int64_t *rhs_shape, int rhs_dim, float *result);
/* :302 reduceSum(axes:) and :280 reduceMax(axis:, context: nil). */
int dl4s_hip_reduce_sum_f32(dl4s_hip_ctx *ctx, const float *values, const int64_t *shape, int dim,
                            const int32_t *axes, int naxes, float *result);
int dl4s_hip_reduce_max_f32(dl4s_hip_ctx *ctx, const float *values, const int64_t *shape, int dim,
                            int axis, float *result);
/* :363 exp, :375 sqrt, :381 relu, :423 tanh */
int dl4s_hip_exp_f32(dl4s_hip_ctx *ctx, const float *values, float *result, int64_t count);
int dl4s_hip_sqrt_f32(dl4s_hip_ctx *ctx, const float *values, float *result, int64_t count);
int dl4s_hip_relu_f32(dl4s_hip_ctx *ctx, const float *values, float *result, int64_t count);
int dl4s_hip_tanh_f32(dl4s_hip_ctx *ctx, const float *values, float *result, int64_t count);
/* :369 log, :393 sin, :399 cos -- the element-wise maps PositionalEncoding (NN/Models/Transformer/
 * PositionalEncoding.swift:52-69) and logSoftmax (Tensor/Operators/Unary.swift:198-204) add to the list */
int dl4s_hip_log_f32(dl4s_hip_ctx *ctx, const float *values, float *result, int64_t count);
int dl4s_hip_sin_f32(dl4s_hip_ctx *ctx, const float *values, float *result, int64_t count);
int dl4s_hip_cos_f32(dl4s_hip_ctx *ctx, const float *values, float *result, int64_t count);
/* :355 argmax(values:count:) -> (index, value): first index of the largest value, NaN never selected, (0, -inf) for an
 * empty buffer (Engine/CPU/Numeric/CPUFloat.swift:294-318).  Synchronises the stream (the result is a host value), as
 * Transformer's greedy decoding needs it (Transformer.swift:130). */
int dl4s_hip_argmax_f32(dl4s_hip_ctx *ctx, const float *values, int64_t count, int64_t *out_index, float *out_value);
/* :478 permuteAxes: source axis i becomes destination axis arrangement[i]
 * (Engine/CPU/CPUEngine.swift:897-935). */
int dl4s_hip_permute_axes_f32(dl4s_hip_ctx *ctx, const float *values, const int64_t *shape, int dim,
                              const int32_t *arrangement, float *result);
/* :493 subscriptRead / :500 subscriptWrite, and the slice forms of MemoryOperatorsType.get(slice:) / set(slice:) (:100-126;
 * semantics Engine/CPU/CPU.swift:137-218): one launch copies the box [start[i], start[i] + extent[i]) of a row-major tensor
 * of shape `shape[dim]` to (read) or from (write) a contiguous buffer of shape `extent`.  An index entry Int i is
 * start = i, extent = 1 (the reference then drops the axis from the result's shape; the layout is the same), nil is
 * start = 0, extent = shape, a range is its lower bound and count.  A pure prefix index needs no copy: it is the offset view
 * of CPU.swift:146-157, plain pointer arithmetic on this side too.  A box that leaves the tensor is DL4S_HIP_ESHAPE. */
int dl4s_hip_subscript_read_f32(dl4s_hip_ctx *ctx, const float *values, const int64_t *shape, int dim, const int64_t *start,
                                const int64_t *extent, float *result);
int dl4s_hip_subscript_write_f32(dl4s_hip_ctx *ctx, const float *values, float *result, const int64_t *shape, int dim,
                                 const int64_t *start, const int64_t *extent);
/* :536 stack along axis 0 of `n` equally shaped buffers of `count` elements each
 * (Tensor/Operators/Stack.swift:79-98 as used by broadcastMatrixMultiplied). */
int dl4s_hip_stack_f32(dl4s_hip_ctx *ctx, const float *const *buffers, int64_t n, int64_t count, float *result);
/* :536 stack along any axis: buffer i is [outer, chunks[i]] (chunks[i] = its extent on the axis times the product of
 * the trailing extents), result is [outer, sum of chunks] (Tensor/Operators/Stack.swift:79-98; PositionalEncoding
 * interleaves sin and cos with it, PositionalEncoding.swift:59-65). */
int dl4s_hip_stack_axis_f32(dl4s_hip_ctx *ctx, const float *const *buffers, const int64_t *chunks, int64_t n, int64_t outer,
                            float *result);

/* ------------------------------------------------ fused layer tails (next to the path) */
/* NN/Layer/LayerNorm.swift:62-77 on x [B, rows, D] -> result, statistics over rows*D jointly per b:
 * mean = sum/N, var = sum(x^2)/N - mean^2, y = (x - mean) * (1 / (sqrt(var) + 1e-5)) * scale + shift.
 * If residual != NULL the input is x + residual (MultiHeadAttention.swift:123-124).
 * The two sums are added in a tree, the reference's reduceSum adds them one after the other
 * (Tensor/Operators/Reduce.swift:106-110).  The one-pass variance cancels when |mean| is large against the standard
 * deviation, and there the order shows: at mean / std = 10 the two differ by 3e-4 relative, and an input whose
 * sequential sums give a negative variance (NaN from the root) may give a small positive one here, or the other way
 * round.  For mean / std up to about 1 - residual sums of normalised activations - the difference is below 1e-6. */
int dl4s_hip_layernorm_f32(dl4s_hip_ctx *ctx, const float *x, const float *residual, const float *scale,
                           const float *shift, float *result, int64_t B, int64_t rows, int64_t D);
/* dl4s_hip_layernorm_f32 with the two sums added in the order the reference's generic CPU engine adds them
 * (Tensor/Operators/Reduce.swift:35-46 -> Engine/CPU/CPUEngine.swift:306-378: reduced = 0, then for every row
 * reduced = reduced + Float.sum(row), Engine/CPU/Numeric/CPUFloat.swift:256-259: dst = 0; dst += src[i] left to right;
 * x * x is rounded before it is added, Reduce.swift:106-110).  Mean, variance and with them every output element are then
 * the reference's to the last bit whatever the input's mean - including the rows where its one-pass variance comes out
 * negative and the root is NaN (NN/Layer/LayerNorm.swift:62-77).  A serial sum cannot be spread over lanes: a lane
 * adds a whole row of D elements, one lane the rows of an item, so the call costs three small launches and a chain of
 * D + rows dependent additions (about 12 us at rows = D = 1024) where dl4s_hip_layernorm_f32 needs two passes.  Same
 * arguments.  The reference built against MKL or Accelerate adds in those libraries' own order, which this does not
 * restate. */
int dl4s_hip_layernorm_reference_order_f32(dl4s_hip_ctx *ctx, const float *x, const float *residual, const float *scale,
                                           const float *shift, float *result, int64_t B, int64_t rows, int64_t D);
/* Tensor/Operators/Unary.swift:245-247: x * (0.5 * tanh(0.5 * (1.702 * x)) + 0.5), optional bias[D] added first
 * (Dense bias, NN/Layer/Dense.swift:64-68). */
int dl4s_hip_bias_gelu_f32(dl4s_hip_ctx *ctx, const float *x, const float *bias, float *result, int64_t rows,
                           int64_t D);
/* Embedding lookup (NN/Layer/Embedding.swift:152-165: row token[t] of the table, a row of zeros for ignore_index)
 * with the rest of Transformer.prepareInputs (Transformer.swift:86-92) folded in when the pointers are given:
 *   result[b][l][:] = row * (*scale) + positions[l][:]
 * table [vocab, D], tokens device int32 [batch, L], positions [L, D] or NULL, scale host pointer or NULL.  Each step
 * is rounded like the separate engine calls.  Token values must lie in [0, vocab) or equal ignore_index (the reference's
 * subscript traps otherwise); the table is never read for a value outside that range: its row of the result is NaN. */
int dl4s_hip_embed_positions_f32(dl4s_hip_ctx *ctx, const float *table, int64_t vocab, int64_t D, const int32_t *tokens,
                                 int64_t batch, int64_t L, int32_t ignore_index, const float *scale, const float *positions,
                                 float *result);
/* logSoftmax over the last axis of x [rows, n] (Tensor/Operators/Unary.swift:198-204): (x - max) - log(sum(exp(x - max))). */
int dl4s_hip_log_softmax_f32(dl4s_hip_ctx *ctx, const float *x, int64_t rows, int64_t n, float *result);
/* The Dense layer with its neighbours folded into the product's epilogue:
 *   result = act(x . weights + bias) + residual
 * x [rows, in], weights [in, out], bias [out] or NULL, residual [rows, out] or NULL, result [rows, out].
 * Dense: NN/Layer/Dense.swift:64-68 (matrixMultiplied, then + bias); activation DL4S_ACT_GELU is
 * gaussianErrorLinear (Tensor/Operators/Unary.swift:245-247) as PointwiseFeedForward applies it to dense1
 * (NN/Models/Transformer/PointwiseFeedForward.swift:75-76); the residual is the `+ denseInputs` of
 * PointwiseFeedForward.swift:79 and the `+ res` of MultiHeadAttention.swift:122 (fc has no bias).  Every step is
 * rounded to fp32 like the separate engine calls, in the same order.  result may alias residual. */
#define DL4S_ACT_NONE 0
#define DL4S_ACT_GELU 1
int dl4s_hip_dense_fused_f32(dl4s_hip_ctx *ctx, const float *x, int64_t rows, int64_t in_features, const float *weights,
                             int64_t out_features, const float *bias, int activation, const float *residual, float *result);
/* The tail of MultiHeadAttention in one call (NN/Models/Transformer/MultiHeadAttention.swift:119-124: the fc product,
 * `+ res`, then norm):
 *   result = LayerNorm(act(x . weights + bias) + residual)
 * with the normalisation of dl4s_hip_layernorm_f32 (NN/Layer/LayerNorm.swift:62-77) over items of item_rows rows
 * (rows % item_rows == 0; item_rows = the sequence length for the reference's joint (L, D) statistics, 1 for per-row
 * ones); scale, shift [out].  When the product runs on the tiled kernels with whole tiles per item, the product's
 * epilogue leaves per-tile sums and sums of squares and one more pass normalises; otherwise the call is
 * dl4s_hip_dense_fused_f32 followed by dl4s_hip_layernorm_f32.  The two routes add the statistics up in different
 * orders and agree to rounding; every element's arithmetic is the same.  result may alias residual. */
int dl4s_hip_dense_layernorm_f32(dl4s_hip_ctx *ctx, const float *x, int64_t rows, int64_t in_features, const float *weights,
                                 int64_t out_features, const float *bias, int activation, const float *residual,
                                 int64_t item_rows, const float *scale, const float *shift, float *result);

#ifdef __cplusplus
}
#endif
#endif /* DL4S_HIP_H */
