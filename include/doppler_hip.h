/*
 * doppler_hip.h -- C ABI of libdopplerhip.so: the MI355X (gfx950) implementation of
 * Doppler's quantized-inference ops.
 *
 * Every entry point below replaces one op of the reference's kernel API
 * (src/gpu/kernels/index.js, re-exported by src/gpu/kernel-selector.js:1-12); the
 * reference function it stands in for is cited on each declaration.  The reference's ops
 * are `runX(...)` / `recordX(recorder, ...)` pairs that enqueue on one GPUQueue; here
 * every op enqueues on one HIP stream (the library's own, which orders itself against
 * the legacy default stream, or the one given to dh_set_stream) and returns at once.
 * Ops never allocate: outputs are caller-provided device pointers, as when the
 * reference's callers pass `outputBuffer`.
 *
 * Conventions
 *   - all pointers named d_* are device pointers (from dh_malloc or any hipMalloc);
 *   - return value 0 = success, non-zero = failure with a message in dh_last_error()
 *     (the reference throws `new Error('[Op] ...')`: the Node addon turns a non-zero
 *     code into exactly such an exception);
 *   - shapes are validated on the host before any launch; an unsupported combination
 *     fails closed (no silent fallback), like src/gpu/kernels/matmul-selection.js:528-539;
 *   - dtype codes: DH_F32 / DH_F16 for activations, Q4_K weights are always the raw
 *     llama.cpp block_q4_K rows the reference's loader uploads
 *     (src/loader/tensors/tensor-loader.js:540-555): W[N,K] = N*ceil(K/256) blocks of
 *     144 bytes, row n at byte n*ceil(K/256)*144.
 */
#ifndef DOPPLER_HIP_H
#define DOPPLER_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DH_F32 0
#define DH_F16 1

#define DH_ACT_SILU 0
#define DH_ACT_GELU 1

#define DH_KV_CONTIGUOUS 0
#define DH_KV_RING 1

/* ---- device, memory, stream (reference: src/gpu/device.js:605-700 initDevice,
 *      src/memory/buffer-pool.js:815-869 acquireBuffer/releaseBuffer/uploadData/readBuffer,
 *      src/gpu/command-recorder.js:499-560 submit/submitAndWait) ---- */
int dh_init(int device_ordinal);
int dh_shutdown(void);
const char* dh_last_error(void);
/* Use a caller-owned hipStream_t for all following ops (NULL: back to the library's). */
int dh_set_stream(void* hip_stream);
void* dh_get_stream(void);
int dh_malloc(size_t bytes, void** d_out);
int dh_free(void* d_ptr);
int dh_upload(void* d_dst, size_t dst_offset, const void* host_src, size_t bytes);
int dh_download(void* host_dst, const void* d_src, size_t src_offset, size_t bytes); /* waits */
int dh_copy(void* d_dst, size_t dst_offset, const void* d_src, size_t src_offset, size_t bytes);
int dh_fill_zero(void* d_dst, size_t offset, size_t bytes);
int dh_sync(void);
/* Timestamps on the op stream (reference: CommandRecorder timestamp-query profiling,
 * src/gpu/command-recorder.js:116-140,728). dh_event_elapsed_ms waits for `stop`. */
int dh_event_create(void** ev_out);
int dh_event_record(void* ev);
int dh_event_elapsed_ms(void* start, void* stop, float* ms_out);
int dh_event_destroy(void* ev);
/* Readback that does not wait for the stream (reference: the ring of token staging buffers that lets a
 * step's token be mapped while later work is queued, src/inference/decode-ring.js:141-177): pinned host
 * memory, a copy enqueued behind the ops so far, and a wait for an event recorded behind that copy.
 * dh_event_synchronize also reports a kernel that gave up a bounded wait, like dh_sync. */
int dh_host_alloc(size_t bytes, void** host_out);
int dh_host_free(void* host_ptr);
int dh_download_async(void* host_dst, const void* d_src, size_t src_offset, size_t bytes);
int dh_event_synchronize(void* ev);

/* ---- captured decode steps ----
 * The reference records a whole decode step into one command encoder and submits it once
 * (src/inference/pipelines/text/generator-steps.js:588-820 decodeStep: recorder at :605, submit at
 * :814; the pre-allocated per-step buffers of src/inference/decode-ring.js make the step replayable).
 * Here: every op enqueued between dh_graph_begin and dh_graph_end is captured into a HIP graph
 * instead of running; dh_graph_launch replays the whole step with one call.  `position` is the
 * token position the captured step was enqueued for; dh_graph_launch(graph, p) first moves the
 * decode attention calls of the step (dh_attn_decode, dh_attn_decode_qkv: start_pos, kv_len, key
 * splits, rotary row, appended cache row) to position p by patching their kernel nodes, everything
 * else (pointers, shapes) replays as captured.  Captured steps must keep at least one key visible.
 * Calls that wait for the stream (dh_upload, dh_download, dh_sync, dh_free) fail during a capture;
 * ops never allocate and dh_fill_zero is a kernel, so nothing in a step is unsuitable for capture. */
int dh_graph_begin(void);
int dh_graph_end(int position, void** graph_out);
int dh_graph_launch(void* graph, int position);
/* A replay at a later position appends further cache rows, reads further rotary rows and may cut the
 * keys into more splits than the captured call did: the caches, the rotary tables and every
 * d_workspace of the captured step must cover the LARGEST position the graph will be launched at
 * (workspaces sized with dh_attn_decode_workspace_bytes for that position's key count).
 * dh_graph_set_max_position declares that position; launches and preparations beyond it then fail
 * with a message instead of writing past those buffers.  (Attention calls that take their key count
 * from device memory, dh_attn_decode_kvlen / dh_attn_decode_qkv_kvlen, carry their own bound and need
 * no patching at all.) */
int dh_graph_set_max_position(void* graph, int max_position);
/* Moves the step to `position` without launching it: a later dh_graph_launch at that position
 * then has nothing left to patch.  Launches already enqueued keep the position they were launched
 * at, so a host can prepare position p + 1 while the GPU still runs position p. */
int dh_graph_prepare(void* graph, int position);
int dh_graph_destroy(void* graph);

/* ---- Q4_K ---- */

/* Dequantize `num_blocks` super-blocks to f32 (bit-exact with
 * tests/kernels/reference/dequant.js:253-300 dequantizeQ4_KBlockRef). */
int dh_q4k_dequant(const void* d_W, int64_t num_blocks, float* d_out);

/* C[M,N] = alpha * A[M,K] . dequant(W)[N,K]^T (+ residual[M,N]).
 * Replaces runMatmul/recordMatmul for Q4_K weights, src/gpu/kernels/matmul.js:659-666
 * (kernels fused_matmul_q4.wgsl:122-258, fused_matmul_q4_batched.wgsl:123-194,
 * fused_matmul_q4_prefill_tiled_f16.wgsl:119-261; f16 activations: fused_matmul_q4_f16a.wgsl,
 * fused_matmul_q4_batched_f16a.wgsl, selected at matmul-selection.js:24-27).  A is f32 or f16
 * (a_dtype); up to 15 f16 rows are loaded as they are by the GEMV kernels and widened (exactly) in registers
 * (K a multiple of 4, rows 8-byte aligned); otherwise they are widened into a 64 MB f32 staging area of the
 * library first, in passes when they do not fit.  The product accumulates in f32 either way.  C is f32 or
 * f16 (c_dtype); the residual is f32.  K need not be a multiple of 256: the padded tail of each row's last
 * block is ignored.  d_residual (may be NULL) is added after alpha, as the reference's
 * `residualTensor` option does.  M = 1..15 takes an HBM-bound GEMV path, M >= 16 the
 * MFMA GEMM path (dh_q4k_matmul_plan tells which kernel family; from 16 rows on a weight tensor must be smaller than 2 GB, as the kernel
 * addresses it through one buffer descriptor; a larger one fails with a message). */
int dh_q4k_matmul(const void* d_A, int a_dtype, const void* d_W, void* d_C, int c_dtype,
                  int M, int N, int K, float alpha, const void* d_residual);

/* dh_q4k_matmul with an RMSNorm prologue: A is replaced by
 * A * rsqrt(mean(A^2 over K) + eps) * (w | 1 + w) row by row before the product, so the
 * standalone norm dispatch in front of the q/k/v and gate/up projections disappears.
 * Replaces runMatmul with `normWeight` + `useFusedRmsnormWideTile`,
 * src/gpu/kernels/matmul-selection.js:609-620 (fused_rmsnorm_q4_widetile.wgsl:4-24,189-215).
 * d_norm_weight is f32 [K].  Below 16 rows the norm runs in the GEMV's prologue (any K; K <= 14336
 * for matrices of more than 61440 rows), from 16 rows on while the GEMM's activations are packed
 * (K <= 16384); longer rows fail with a message (run dh_rmsnorm + dh_q4k_matmul). */
int dh_q4k_matmul_rmsnorm(const float* d_A, const float* d_norm_weight, float eps,
                          int weight_offset, const void* d_W, void* d_C, int c_dtype, int M,
                          int N, int K, float alpha, const void* d_residual);

/* Which kernel family dh_q4k_matmul / dh_q4k_matmul_rmsnorm (dual = 0) or dh_q4k_ffn_gate_up[_rmsnorm]
 * (dual = 1; N = intermediate size, K = hidden size) takes for f32 activations of this shape, without
 * launching anything: the dispatch of src/gpu/kernels/matmul-selection.js:427-667
 * selectMatmulVariantAndFlags made visible.  Needs no device: num_cus is the compute-unit count to
 * plan for (<= 0: the initialised device's, or 256).  Returns a DH_PLAN_* family, or 0 with a message
 * in dh_last_error() when no kernel serves the shape. */
#define DH_PLAN_GEMV_I8 1    /* M <= 2: int8 matrix cores, activations as block fixed point */
#define DH_PLAN_GEMV_ROWS 2  /* M = 3..15: f16 matrix cores, one sweep over the weights per 8 rows */
#define DH_PLAN_GEMV_RING 3  /* few work units per workgroup: a tile's columns spread over the waves */
#define DH_PLAN_GEMM 4       /* M >= 16: f16 matrix-core GEMM */
#define DH_PLAN_GEMV_LDS 5   /* f32 vector GEMV, activations staged in LDS: last resort */
int dh_q4k_matmul_plan(int M, int N, int K, int normed, int dual, int num_cus);
/* dh_q4k_matmul_plan plus, for the two streaming GEMV families, the launch the call would make (its
 * first pass): out12 = { weight rows per tile, load instructions per work unit, workgroups, tiles per
 * workgroup (floor), workgroups with one tile more, ring stages per wave, bytes of dynamic LDS,
 * int8 kernel: work units per tile, its reciprocal multiplier, tile slots; few-row kernel:
 * accumulators per wave; activation rows per pass }.  For tests that check the kernels' address
 * arithmetic on the host; other families leave the record zero.  No counterpart in the reference. */
int dh_q4k_gemv_layout(int M, int N, int K, int normed, int dual, int num_cus, int64_t* out12);

/* out[M,inter] = clamp(act(x.Wgate^T) * (x.Wup^T) * alpha).
 * Replaces runFusedFFN/recordFusedFFN, src/gpu/kernels/fused_ffn.js:501,605
 * (fused_ffn_q4k.wgsl:129-363).  clamp (swigluLimit) applies to DH_ACT_SILU only;
 * 0 disables it. */
int dh_q4k_ffn_gate_up(const float* d_x, const void* d_Wgate, const void* d_Wup, float* d_out,
                       int M, int hidden, int inter, int activation, float alpha,
                       float swiglu_limit);

/* dh_q4k_ffn_gate_up over RMSNorm(x): the reference's "fused normed FFN",
 * src/gpu/kernels/fused_ffn.js:705-745,773-860 (there the inverse RMS comes in as a buffer,
 * here it is computed in the prologue).  d_norm_weight is f32 [hidden]; limits as for
 * dh_q4k_matmul_rmsnorm. */
int dh_q4k_ffn_gate_up_rmsnorm(const float* d_x, const float* d_norm_weight, float eps,
                               int weight_offset, const void* d_Wgate, const void* d_Wup,
                               float* d_out, int M, int hidden, int inter, int activation,
                               float alpha, float swiglu_limit);

/* ---- chained decode products ----
 * Up to DH_CHAIN_MAX_PHASES dependent Q4_K products of ONE activation row in a single launch:
 *     x_0 = d_x0,   x_{p+1} = f_p( W_p . g_p(x_p) ),   C_p = x_{p+1}
 * g_p: RMSNorm of the product's input when d_norm_weight is set (as in dh_q4k_matmul_rmsnorm);
 * f_p: alpha * (.) + residual (as dh_q4k_matmul), or with d_W2 the gated pair
 * act(W . x) * (W2 . x) * alpha (as dh_q4k_ffn_gate_up).  The reference records these products one
 * after the other into the step's command encoder (src/inference/pipelines/text/layer.js:682
 * processLayerGPU -> attention/interpreter.js:1148 o_proj, ffn/dense.js:727 gate/up and down, then
 * the next layer's attention/projections.js:641 q/k/v) and submits once per token
 * (generator-steps.js:814); here the run between two attentions is one persistent launch in which
 * the weight stream of a product starts while the previous product's outputs still travel between
 * the workgroups.  Results equal those of the separate calls (same kernels' arithmetic).
 * Limits: K of every product a multiple of 256 and at least 2048, N and K at most 32768,
 * K_p = N_{p-1}, f32 vectors, 16-byte aligned pointers; a product's d_residual may be an earlier
 * product's d_C (or d_x0's producer's output), d_C must not be d_x0.  Launches are ordered on the
 * op stream and share one exchange area of the library: one chain at a time per device.
 * Every wait inside the launch is bounded: if one gives up (it cannot while the launch has the
 * device's compute units to itself) all waves exit, the outputs are undefined, and the next call
 * that waits for the stream (dh_sync, dh_download, dh_upload, dh_free) fails with the reason. */
#define DH_CHAIN_MAX_PHASES 4
typedef struct dh_chain_phase {
  const void* d_W;             /* Q4_K [N,K] */
  const void* d_W2;            /* second matrix of a gated pair (the "up" rows), or NULL */
  float* d_C;                  /* [N] f32 */
  const float* d_residual;     /* [N] f32 or NULL (not with d_W2) */
  const float* d_norm_weight;  /* [K] f32 or NULL */
  int N, K;
  int activation;              /* DH_ACT_*, used with d_W2 */
  int norm_weight_offset;      /* 1: weights are 1 + w */
  float alpha;
  float swiglu_limit;          /* clamp of the gated pair's output (DH_ACT_SILU only); 0 = off */
  float norm_eps;
} dh_chain_phase;
int dh_q4k_gemv_chain(const float* d_x0, const dh_chain_phase* phases, int n_phases);
/* Diagnostic form: launches only the first `workgroups` workgroups of the chain and bounds every
 * wait at `spin_limit` polls.  With fewer workgroups than compute units the missing ones' outputs
 * never arrive, so the waits give up, every wave exits, and the next synchronising call reports
 * it: the way to exercise the failure path without hanging anything.  No counterpart in the
 * reference. */
int dh_q4k_gemv_chain_limited(const float* d_x0, const dh_chain_phase* phases, int n_phases,
                              int workgroups, int spin_limit);
/* dh_q4k_gemv_chain whose first product reads the attention output of the step: the merge of the
 * split-K partial results that dh_attn_decode_qkv_partials / dh_attn_decode_qkv_kvlen_partials left
 * in their workspace (the arithmetic of the attention's own merge, same bits), done inside the
 * launch by one wave per query head and handed to every workgroup through the chain's exchange.
 * H * D must be the first product's K; at most 64 key splits.  d_kv_len NULL: nsplit is the count
 * dh_attn_decode_qkv_partials returned; else the key count is read on the device and max_kv_len,
 * sliding_window and kv_start are those given to dh_attn_decode_qkv_kvlen_partials. */
typedef struct dh_chain_attn_source {
  const void* d_workspace;
  int H, Hkv, D;
  int nsplit;
  const uint32_t* d_kv_len;
  int max_kv_len, sliding_window, kv_start;
} dh_chain_attn_source;
int dh_q4k_gemv_chain_attn(const dh_chain_attn_source* source, const dh_chain_phase* phases, int n_phases);
/* 1 when dh_q4k_gemv_chain_attn serves this head geometry for key counts up to max_kv_len on the
 * current device (after dh_init), else 0. */
int dh_q4k_gemv_chain_attn_supported(int H, int Hkv, int D, int max_kv_len);

/* ---- dense f16-weight GEMV (LM head) ----
 * C[M,N] = alpha * A[M,K] . f32(W[N,K])^T, W row-major f16.  Replaces the f16-weight branch
 * of runMatmul (matmul_gemv_subgroup.wgsl) used by recordLogitsGPU,
 * src/inference/pipelines/text/logits/gpu.js:1122-1157. */
int dh_f16w_matmul(const float* d_A, const void* d_W, float* d_C, int M, int N, int K,
                   float alpha);

/* Final-logit GEMV fused with greedy argmax: token = argmax_v softcap(h . E[v,:]).
 * Replaces recordLmHeadArgmaxF16, src/gpu/kernels/lm-head-argmax.js:304-315
 * (lm_head_argmax_f16.wgsl:53-147).  Ties go to the lowest index; pad_token_id < 0 = none.
 * d_workspace needs dh_lmhead_argmax_workspace_bytes(vocab) bytes; d_logits_out may be NULL. */
size_t dh_lmhead_argmax_workspace_bytes(int vocab);
int dh_lmhead_argmax_f16(const float* d_h, const void* d_E, int vocab, int hidden,
                         int64_t pad_token_id, float logit_softcap, void* d_workspace,
                         uint32_t* d_token_out, int output_index, float* d_logits_out);
/* The same over RMSNorm(h) (weight f32 [hidden], w or 1 + w), the norm done on the row in the GEMV's
 * registers: recordLogitsGPU's final norm + LM head (src/inference/pipelines/text/logits/gpu.js:1122-1157)
 * fused with recordLmHeadArgmaxF16 into one call.  hidden <= 4096, h and the weight 16-byte aligned;
 * other shapes fail with a message (run dh_rmsnorm in front of dh_lmhead_argmax_f16 there). */
int dh_lmhead_argmax_f16_rmsnorm(const float* d_h, const float* d_norm_weight, float eps, int weight_offset,
                                 const void* d_E, int vocab, int hidden, int64_t pad_token_id,
                                 float logit_softcap, void* d_workspace, uint32_t* d_token_out,
                                 int output_index, float* d_logits_out);

/* ---- attention ----
 * Decode attention of one query token over an f16 KV cache.  Replaces
 * runAttention/recordAttention for seqLen == 1, src/gpu/kernels/attention.js:2007-2030
 * (attention_decode_online_f16kv.wgsl:84-243).  Q f32 [H][D], K/V f16 [pos][Hkv][D],
 * O f32 [H][D].  kv_layout DH_KV_RING reads row (kv_start+k) % sliding_window.
 * d_workspace needs dh_attn_decode_workspace_bytes(H, D, kv_len) bytes (split-K partials). */
size_t dh_attn_decode_workspace_bytes(int H, int D, int kv_len);
/* Prefill attention: T query tokens (Q f32 [T][H][D], already rotated) against the f16 cache rows
 * [0, kv_len), query t at absolute position start_pos + t; causal and sliding-window masks as in
 * the decode op; contiguous cache layout.  Replaces runAttention/recordAttention for seqLen > 1,
 * src/gpu/kernels/attention.js:1047-1310 (attention_streaming_f16kv.wgsl and the tiled prefill
 * variants).  Scores and P.V run on the matrix cores with f16 inputs and f32 accumulation. */
int dh_attn_prefill(const float* d_Q, const void* d_K, const void* d_V, float* d_O, int T, int H,
                    int Hkv, int D, int kv_len, float scale, int causal, int start_pos,
                    float softcap, int sliding_window);
int dh_attn_decode(const float* d_Q, const void* d_K, const void* d_V, float* d_O, int H,
                   int Hkv, int D, int kv_len, float scale, int causal, int start_pos,
                   float softcap, int sliding_window, int kv_start, int kv_layout,
                   void* d_workspace);
/* dh_attn_decode for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): the split-K partials go to a fixed 4 MiB
 * device array inside the library instead of a caller's workspace, and the call allocates nothing.
 * It has no counterpart in the reference.  Arguments and results as dh_attn_decode; a shape whose
 * partials (numHeads * key splits * (headDim + 2) floats) exceed
 * dh_attn_decode_static_max_bytes() fails with a message.  Every call on a GPU shares that GPU's
 * array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not. */
size_t dh_attn_decode_static_max_bytes(void);
int dh_attn_decode_static(const float* d_Q, const void* d_K, const void* d_V, float* d_O, int H,
                          int Hkv, int D, int kv_len, float scale, int causal, int start_pos,
                          float softcap, int sliding_window, int kv_start, int kv_layout);
/* One decode step's attention straight from the stacked projection qkv[(H+2Hkv)*D] (f32): per-head
 * RMSNorm (use_norm) and rotary embedding of q and k, k and v narrowed to f16 and appended to the
 * caches at the row of start_pos, then causal attention of the new token over rows up to and
 * including its own.  Same results as dh_qkv_norm_rope_kvwrite (T = 1, dst row of start_pos)
 * followed by dh_attn_decode (kv_len = start_pos - kv_start + 1, causal), in one launch fewer;
 * i.e. recordSplitQKVRMSNormRoPEQK with f16KVCacheWrite,
 * src/gpu/kernels/split-qkv-rmsnorm-rope-qk.js:244-250, followed by recordAttention for
 * seqLen == 1, src/gpu/kernels/attention.js:2007-2030.  d_cos/d_sin are the whole tables
 * [max_seq][rotary_dim/2].  dh_attn_decode_qkv_supported tells whether a head geometry is served
 * (head_dim 64 or 128; rotary_dim even when interleaved, else a power of two of at least
 * head_dim/16); workspace as for dh_attn_decode. */
int dh_attn_decode_qkv_supported(int H, int Hkv, int D, int rotary_dim, int interleaved);
int dh_attn_decode_qkv(const float* d_qkv, const float* d_q_weight, const float* d_k_weight,
                       const float* d_cos, const float* d_sin, void* d_cache_k, void* d_cache_v,
                       float* d_O, int H, int Hkv, int D, int start_pos, int rotary_dim,
                       int interleaved, float eps, int weight_offset, int use_norm, float scale,
                       float softcap, int sliding_window, int kv_start, int kv_layout,
                       void* d_workspace);

/* ---- decode attention with the key count in device memory ----
 * The reference's `kvLenBuffer` option of runAttention (src/gpu/kernels/attention.js:1071,1224-1232;
 * attention_decode_online_f16kv.wgsl:27,39,55-58 get_kv_len with kv_len_source == 1): the number of
 * cached keys is read by the kernels from a u32 in device memory, so a recorded decode step can be
 * replayed for the next token without touching its launch arguments.  d_kv_len points at that
 * word; max_kv_len bounds it (larger values are clamped): the caches, the rotary tables and
 * d_workspace (dh_attn_decode_workspace_bytes(H, D, max_kv_len), always required) must cover it,
 * and the launch holds the key splits of max_kv_len, of which the surplus exits at once.
 * dh_attn_decode_kvlen: start_pos >= 0 is the query's position as in dh_attn_decode; start_pos < 0
 * places the query at the last key, kv_start + kv_len - 1 (what a decode step means).  A key count of
 * zero gives a zero output.
 * dh_attn_decode_qkv_kvlen: dh_attn_decode_qkv for the token at position kv_start + kv_len - 1 (its
 * rotary row, its appended cache row); the key count must be at least 1. */
int dh_attn_decode_kvlen(const float* d_Q, const void* d_K, const void* d_V, float* d_O, int H, int Hkv,
                         int D, const uint32_t* d_kv_len, int max_kv_len, float scale, int causal,
                         int start_pos, float softcap, int sliding_window, int kv_start, int kv_layout,
                         void* d_workspace);
int dh_attn_decode_qkv_kvlen(const float* d_qkv, const float* d_q_weight, const float* d_k_weight,
                             const float* d_cos, const float* d_sin, void* d_cache_k, void* d_cache_v,
                             float* d_O, int H, int Hkv, int D, const uint32_t* d_kv_len,
                             int max_kv_len, int rotary_dim, int interleaved, float eps,
                             int weight_offset, int use_norm, float scale, float softcap,
                             int sliding_window, int kv_start, int kv_layout, void* d_workspace);
/* dh_attn_decode_qkv / dh_attn_decode_qkv_kvlen without the merge of the key splits: the splits'
 * partial results stay in the workspace, [H][S][D + 2] floats (unnormalised output, running
 * maximum, running sum per query head and split; S = the split count, or with the key count on the
 * device the largest count any key count up to max_kv_len can ask for), for a consumer that merges them itself
 * (dh_q4k_gemv_chain_attn: the reference's single attention dispatch,
 * src/gpu/kernels/attention_decode_online_f16kv.wgsl:84-243, followed by its o-projection,
 * src/inference/pipelines/text/attention/interpreter.js:1121-1160, with the launch between them removed).
 * dh_attn_decode_qkv_partials hands back the split count of this position (not while a graph is
 * being captured); with the key count on the device the consumer derives it from the same word. */
int dh_attn_decode_qkv_partials(const float* d_qkv, const float* d_q_weight, const float* d_k_weight,
                                const float* d_cos, const float* d_sin, void* d_cache_k, void* d_cache_v,
                                int H, int Hkv, int D, int start_pos, int rotary_dim, int interleaved,
                                float eps, int weight_offset, int use_norm, float scale, float softcap,
                                int sliding_window, int kv_start, int kv_layout, void* d_workspace,
                                int* out_nsplit);
int dh_attn_decode_qkv_kvlen_partials(const float* d_qkv, const float* d_q_weight, const float* d_k_weight,
                                      const float* d_cos, const float* d_sin, void* d_cache_k,
                                      void* d_cache_v, int H, int Hkv, int D, const uint32_t* d_kv_len,
                                      int max_kv_len, int rotary_dim, int interleaved, float eps,
                                      int weight_offset, int use_norm, float scale, float softcap,
                                      int sliding_window, int kv_start, int kv_layout, void* d_workspace);

/* ---- normalisation / rotary / KV ---- */

/* y = x' * rsqrt(mean(x'^2)+eps) * (w | 1+w) [+ post_residual] * output_scale with
 * x' = x (+ pre_residual); optional side output prenorm_out = x'.  Replaces
 * runRMSNorm/recordRMSNorm, src/gpu/kernels/rmsnorm.js:146-297 (rmsnorm.wgsl:120-187).
 * weight_dtype DH_F32 or DH_F16; d_weight NULL = all ones. */
int dh_rmsnorm(const float* d_x, const void* d_weight, int weight_dtype, float* d_out,
               int batch, int hidden, float eps, int weight_offset, const float* d_pre_residual,
               const float* d_post_residual, float* d_prenorm_out, float output_scale);

/* Per-head RMSNorm of q [q_rows, head_dim] and k [k_rows, head_dim] in one launch, each with its
 * own weight [head_dim] (f32 or f16; 1 + w with weight_offset).  Replaces
 * runRMSNormQK/recordRMSNormQK, src/gpu/kernels/rmsnorm-qk.js:122-128 (rmsnorm_qk.wgsl:74-118);
 * q_rows = numTokens * numHeads, k_rows = numTokens * numKVHeads.  Outputs may alias the inputs. */
int dh_rmsnorm_qk(const float* d_q, const float* d_k, const void* d_q_weight, int q_weight_dtype,
                  const void* d_k_weight, int k_weight_dtype, float* d_q_out, float* d_k_out,
                  int q_rows, int k_rows, int head_dim, float eps, int weight_offset);

/* post = rmsnorm(x, post_weight) (+ residual, may be NULL); pre = rmsnorm(post, pre_weight), one
 * launch.  Replaces runSandwichRMSNormPair/recordSandwichRMSNormPair,
 * src/gpu/kernels/rmsnorm-pair.js:147-167 (rmsnorm_pair.wgsl:4-5,109-166).  d_post_out may alias
 * d_x or d_residual (each element is read before it is written); the two outputs must differ. */
int dh_rmsnorm_sandwich_pair(const float* d_x, const float* d_residual, const void* d_post_weight,
                             int post_weight_dtype, const void* d_pre_weight, int pre_weight_dtype,
                             float* d_post_out, float* d_pre_out, int batch, int hidden, float eps,
                             int weight_offset);

/* residual_out = (x + residual) * output_scale; norm_out = rmsnorm(residual_out, norm_weight), one
 * launch.  Replaces runResidualNextRMSNormPair/recordResidualNextRMSNormPair,
 * src/gpu/kernels/rmsnorm-pair.js:246-266 (residual_rmsnorm_pair.wgsl:75-119). */
int dh_residual_rmsnorm_pair(const float* d_x, const float* d_residual, const void* d_norm_weight,
                             int norm_weight_dtype, float* d_residual_out, float* d_norm_out, int batch,
                             int hidden, float eps, int weight_offset, float output_scale);

/* In-place rotary embedding on x[seq][heads][head_dim] with host-built tables
 * cos/sin[max_seq][rotary_dim/2].  Replaces runRoPE/recordRoPE,
 * src/gpu/kernels/rope.js:108-114 (rope.wgsl:63-106). */
int dh_rope(float* d_x, const float* d_cos, const float* d_sin, int seq, int heads,
            int head_dim, int rotary_dim, int pair_span_dim, int interleaved, int start_pos);

/* In-place rotary embedding of q[seq][q_heads][head_dim] and k[seq][kv_heads][head_dim] in one
 * launch, same tables and pairing rules as dh_rope; seq == 0 is a no-op.  Replaces
 * runRoPEQK/recordRoPEQK, src/gpu/kernels/rope-qk.js:67-143 (rope_qk.wgsl:41-95). */
int dh_rope_qk(float* d_q, float* d_k, const float* d_cos, const float* d_sin, int seq, int q_heads, int kv_heads,
               int head_dim, int rotary_dim, int pair_span_dim, int interleaved, int start_pos);

/* From fused qkv[T][(H+2Hkv)*D]: per-head RMSNorm (q/k weights) -> RoPE -> Q out f32,
 * K and V narrowed to f16 straight into the caches at element kv_dst_offset.  Replaces
 * recordSplitQKVRMSNormRoPEQK with f16KVCacheWrite,
 * src/gpu/kernels/split-qkv-rmsnorm-rope-qk.js:244-250
 * (split_qkv_rmsnorm_rope_qk_f16kv_cache.wgsl:168-217).  use_norm 0 skips the RMSNorm
 * (plain RoPE + KV write, i.e. recordRoPE x2 + recordKVCacheWriteF32ToF16). */
int dh_qkv_norm_rope_kvwrite(const float* d_qkv, const float* d_q_weight, const float* d_k_weight,
                             const float* d_cos, const float* d_sin, float* d_q_out,
                             void* d_cache_k, void* d_cache_v, int T, int H, int Hkv, int D,
                             int start_pos, int rotary_dim, int interleaved, float eps,
                             int weight_offset, int64_t kv_dst_offset, int use_norm);

/* cache[dst+i] = f16(src[src_off+i]) for K and V.  Replaces
 * runKVCacheWriteF32ToF16, src/gpu/kernels/kv-cache-write.js:107-126
 * (kv_cache_write_f32_to_f16.wgsl:18-32). */
int dh_kv_write_f16(const float* d_k, const float* d_v, void* d_cache_k, void* d_cache_v,
                    int64_t src_offset, int64_t dst_offset, int64_t count);

/* ---- elementwise glue ---- */

/* out = (a + b) * scale.  Replaces runResidualAdd, src/gpu/kernels/residual.js:210-216
 * (residual.wgsl:24-31). */
int dh_residual_add(const float* d_a, const float* d_b, float* d_out, int64_t n, float scale);

/* Rows of qkv[num_tokens][q_size + k_size + v_size] copied apart into q[num_tokens][q_size],
 * k[num_tokens][k_size], v[num_tokens][v_size].  Replaces runSplitQKV/recordSplitQKV,
 * src/gpu/kernels/split_qkv.js:6-45. */
int dh_split_qkv(const float* d_qkv, float* d_q, float* d_k, float* d_v, int num_tokens, int q_size, int k_size,
                 int v_size);

/* data[t][d] += bias[d] in place for t < num_tokens, d < dim; the byte offsets select the start
 * inside each buffer; bias is DH_F32 or DH_F16.  Replaces runBiasAdd/recordBiasAdd,
 * src/gpu/kernels/residual.js:165-224 (bias_add.wgsl:27-39). */
int dh_bias_add(float* d_data, const void* d_bias, int bias_dtype, int64_t num_tokens, int dim,
                int64_t data_offset_bytes, int64_t bias_offset_bytes);

/* out = in * scale over n elements; d_out may equal d_in (the reference's inplace variant).
 * Replaces runScale/recordScale, src/gpu/kernels/scale.js:13-46. */
int dh_scale(const float* d_in, float* d_out, int64_t n, float scale);

/* out[t,:] = f32(E[ids[t + index_offset], :]) (zero row when the id is outside the
 * vocabulary).  Replaces runGather for f16 tables, src/gpu/kernels/gather.js:370-391
 * (gather_f16.wgsl:35-66). */
int dh_gather_f16(const uint32_t* d_ids, const void* d_table, float* d_out, int T, int hidden,
                  int vocab, int index_offset);

/* out = clamp(act(gate) * up).  Replaces runSiLU with `gate` (src/gpu/kernels/silu.js:95,
 * silu.wgsl:100-106) and runGeLU with `gate` (gelu.wgsl:60-65). */
int dh_act_gate(const float* d_gate, const float* d_up, float* d_out, int64_t n, int activation,
                float swiglu_limit);

/* Row-split form: in[T][2*dim] -> out[T][dim].  Replaces runSiLURowSplit,
 * src/gpu/kernels/silu.js:230-288 (silu.wgsl:83-98, gelu.wgsl:37-52). */
int dh_act_gate_rowsplit(const float* d_in, float* d_out, int T, int dim, int activation,
                         float swiglu_limit);

/* Greedy argmax over f32 logits, ties to the lowest index, optional pad id (<0: none) and
 * soft cap.  Replaces runArgmax/recordArgmax, src/gpu/kernels/sample.js:258-341
 * (sample.wgsl:311-400).  d_workspace needs dh_argmax_workspace_bytes() bytes. */
size_t dh_argmax_workspace_bytes(void);
int dh_argmax(const float* d_logits, int vocab, int64_t pad_token_id, float logit_softcap,
              void* d_workspace, uint32_t* d_token_out, int output_index);

/* Top-k temperature sampling: the top_k (<= 256) logits by value (ties to the lower index),
 * softmax of value / temperature over them, first candidate whose running probability reaches
 * random_value.  Replaces runGPUSample/recordGPUSample, src/gpu/kernels/sample.js:343-568
 * (sample.wgsl:66-243), with the selection of the reference's sampler oracle
 * (tests/kernels/reference/sample.js:62-92: exact top-k; the WGSL keeps one candidate per
 * workgroup).  The caller draws random_value (seededRandom, sample.js:569-572) and routes
 * temperature below its greedy threshold to dh_argmax.  d_workspace needs
 * dh_sample_topk_workspace_bytes(vocab, top_k) bytes. */
size_t dh_sample_topk_workspace_bytes(int vocab, int top_k);
int dh_sample_topk(const float* d_logits, int vocab, double temperature, int top_k,
                   double random_value, int64_t pad_token_id, float logit_softcap,
                   void* d_workspace, uint32_t* d_token_out, int output_index);

/* f32 <-> f16 casts.  Replaces castF32ToF16/castF16ToF32, src/gpu/kernels/cast.js:98-116. */
int dh_cast_f32_to_f16(const float* d_in, void* d_out, int64_t n);
int dh_cast_f16_to_f32(const void* d_in, float* d_out, int64_t n);

/* out[n] = y[n] / sqrt(mean(y^2 over N) + eps) * (w[n] | 1 + w[n]) (+ residual[n]) with
 * y = x[1,K] . W, W dense f32 laid out [N,K] (transpose_b != 0) or [K,N].  Replaces
 * runMatmulRMSNormFused/recordMatmulRMSNormFused, src/gpu/kernels/fused_matmul_rmsnorm.js:50-170
 * and :173-296 (fused_matmul_rmsnorm.wgsl:166-213, :215-272): one activation row, N <= 4096
 * (the reference's maxMediumN; larger N fails with its message), norm weight f32 or f16, the
 * residual added after the norm.  Uses the library's split-K workspace: two or three launches
 * on the library's stream, the product over the whole chip in K slices, the sum of the slices
 * when there are many, and the row's norm in one workgroup. */
int dh_matmul_rmsnorm_f32(const float* d_x, const float* d_W, int transpose_b,
                          const void* d_norm_weight, int norm_weight_dtype, float eps,
                          int weight_offset, const float* d_residual, float* d_out, int N, int K);
/* The same with f16 activations, weights, residual and output (the reference's small_f16 /
 * medium_f16 variants, fused_matmul_rmsnorm_f16.wgsl): every sum runs in f32 and the result is
 * rounded to f16 once, on the final store. */
int dh_matmul_rmsnorm_f16(const void* d_x, const void* d_W, int transpose_b,
                          const void* d_norm_weight, int norm_weight_dtype, float eps,
                          int weight_offset, const void* d_residual, void* d_out, int N, int K);

/* Overflow guard for activations: the first element of d_input (f32 or f16) that is NaN,
 * infinite or larger in magnitude than abs_threshold (<= 0 or not finite: 65500) turns
 * d_status[0] from 0 to 1, and the launch that does so writes layer to d_status[1] and step to
 * d_status[2]; a status that is already 1 is left alone.  d_status is 4 u32 words the caller
 * zeroes before a step and reads back beside the token.  Replaces recordCheckFiniteness,
 * src/gpu/kernels/check-finiteness.js:98-150 (shader :25-62); read back as the reference does at
 * src/inference/pipelines/text/generator-steps.js:786-798.  Recorded into a captured step
 * (dh_graph_begin .. dh_graph_end) its step number follows the replay position:
 * step + position - position of the capture. */
int dh_check_finiteness(const void* d_input, int dtype, int64_t size, uint32_t* d_status,
                        uint32_t layer, uint32_t step, float abs_threshold);

#ifdef __cplusplus
}
#endif
#endif /* DOPPLER_HIP_H */
