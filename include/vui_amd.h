/*
 * vui_amd.h - C ABI of the MI355X (gfx950) decode-step library for Vui.
 *
 * The reference has no native boundary for this path: its "operator API" is the Python
 * surface of src/vui/model.py and src/vui/engine.py, whose GPU arithmetic is delegated to
 * torch/cuBLAS, flash_attn_with_kvcache and torch.cuda.CUDAGraph.  Each entry point below
 * names the reference call it stands in for.  All pointers marked "device" are HIP device
 * pointers; the library never allocates or frees device memory: buffers (weights, KV caches,
 * workspace, outputs) are owned by the caller.  Work is enqueued on the given stream without
 * waiting for it, and the per-step calls may be recorded into a HIP graph; the exceptions are
 * vui_ctx_init and vui_ctx_status, which wait for the stream / the device (said at each).
 *
 * Persistent kernels: the batch-1 frame kernel, the batched depth head and the vocoder's trunk
 * kernel keep one workgroup resident on every compute unit and hand values to each other
 * while they run.  While such a launch is in flight NO other kernel may run on the device
 * (another stream, another context, another process): a workgroup kept off its compute unit
 * makes the others wait until a bounded spin gives up; the launch then raises the context's
 * error word, and vui_ctx_status reports VUI_EHIP until the context is initialised again with
 * vui_ctx_init.  The batch-1 frame kernel commits nothing in that case (no position update, no
 * repetition state, no codes; its EOS probability reads -1).  The batched kernels (depth head and
 * backbone step of 2..16 rows) and the vocoder's trunk kernel write their output buffers as they
 * go: after a failed launch those hold unfinished values, which a caller must discard - so a caller
 * checks vui_ctx_status before it uses what such launches wrote (the position update of a batched
 * backbone step is withheld like the frame kernel's).
 *
 * Return value: 0 on success, a negative VUI_E* code on failure; vui_last_error() returns a
 * human-readable description of the last failure on the calling thread.
 */
#ifndef VUI_AMD_H
#define VUI_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VUI_OK 0
#define VUI_EINVAL (-22)  /* bad argument / unsupported shape */
#define VUI_EHIP (-5)     /* a HIP runtime call failed */
#define VUI_ENOMEM (-12)  /* workspace too small */

#define VUI_DTYPE_BF16 0
#define VUI_DTYPE_F32 1

#define VUI_MAX_LAYERS 64
#define VUI_MAX_RQ_LAYERS 16
#define VUI_MAX_BATCH 16

typedef void* vui_stream_t; /* hipStream_t */

/* Architecture numbers; mirrors VuiConfig (src/vui/config.py:16-52) as consumed by
 * Vui.__init__ (src/vui/model.py:1061-1136). */
typedef struct vui_config {
  int32_t dtype;          /* VUI_DTYPE_*: element type of weights, activations and KV caches */
  int32_t d_model, n_layers, n_heads, n_kv_heads, head_dim, ffn;
  int32_t n_quantizers, codebook_size;
  int32_t rq_dim, rq_layers, rq_heads, rq_ffn;
  int32_t rope_dim;       /* leading features of each head that are rotated (<= head_dim, even) */
  int32_t max_seqlen;     /* S of the KV caches and of the RoPE table */
  int32_t n_slots;        /* KV cache slots (reference: max_rows + 1, engine.py:380-387) */
  int32_t window;         /* sliding window of every layer, 0 = full attention (model.py:256) */
  float norm_eps;         /* backbone RMSNorm eps (model.py:391) */
  float rq_norm_eps;      /* RQ RMSNorm eps (model.py:287) */
  int32_t int8_backbone;  /* 1: backbone linears are int8 weight-only with per-row scales */
  /* Global-attention layers (Decoder's window_size / global_every / global_rope_*, model.py:396-468): bit l set =
   * layer l attends over the whole cache whatever `window` says and, when vui_weights.rope_table_global is given,
   * rotates with that table over its first global_rope_dim features.  0 = every layer as configured above. */
  uint64_t global_layers;
  int32_t global_rope_dim; /* rotated features of the global table (<= head_dim, even); used with rope_table_global */
  int32_t reserved;
} vui_config;

/* One backbone block (src/vui/model.py:300-340).  nn.Linear layout (out, in), row-major. */
typedef struct vui_layer_weights {
  const void* attn_norm;  /* (d) */
  const void* wqkv;       /* ((H+2KV)*hd, d)   dtype, or int8 when int8_backbone */
  const void* wo;         /* (d, d) */
  const void* mlp_norm;   /* (d) */
  const void* w1;         /* (ffn, d) */
  const void* w3;         /* (ffn, d) */
  const void* w2;         /* (d, ffn) */
  /* per-output-row scales (dtype elements) when int8_backbone, else NULL */
  const void *s_qkv, *s_o, *s_1, *s_3, *s_2;
} vui_layer_weights;

/* One RQ block (src/vui/model.py:577-597). */
typedef struct vui_rq_layer_weights {
  const void *attn_norm, *wqkv, *wo, *mlp_norm, *w1, *w3, *w2;
} vui_rq_layer_weights;

typedef struct vui_weights {
  const void* audio_emb;    /* (Q*CS, d)   model.py:552-563 */
  const void* final_norm;   /* (d)         decoder.norm */
  const void* codec_head;   /* (CS, d)     model.py:1083 */
  const void* eos_w;        /* (1, d)      model.py:1099 */
  const void* eos_b;        /* (1) */
  const float* rope_table;  /* (max_seqlen, rope_dim, 2) fp32 cos/sin, rope.py:60-77 */
  vui_layer_weights layers[VUI_MAX_LAYERS];
  const void* rq_backbone_proj; /* (R, d) or NULL when R == d (nn.Identity, model.py:653-657) */
  const void* rq_code_emb;      /* ((Q-1)*CS, R) */
  const void* rq_pos_emb;       /* (Q, R) */
  const void* rq_head_w;        /* (Q-1, CS, R) */
  const void* rq_norm;          /* (R) */
  vui_rq_layer_weights rq_layers[VUI_MAX_RQ_LAYERS];
  const float* rope_table_global; /* (max_seqlen, global_rope_dim, 2) fp32 cos/sin of the global layers' own
                                     table (Decoder.freqs_cis_global, model.py:449-468), or NULL: they use rope_table */
} vui_weights;

typedef struct vui_ctx vui_ctx;

const char* vui_last_error(void);
int vui_version(void);

/* Bytes of device workspace a context needs for up to max_batch rows.  For a configuration that has the one-pass
 * prompt ingestion (vui_prefill) this includes a second copy of the layers' projection weights in the operand
 * layout of its GEMMs (Vui Nano: 311 MB), and for one that has the batched depth-head kernel a copy of the depth
 * head's matrices in that kernel's layout (58 MB); for a configuration that has the batched backbone kernel a copy of the codec head in its layout
 * and, with int8 weights, of the layers' int8 matrices (Vui Nano: 3 + 156 MB).  All are written by vui_ctx_init. */
int64_t vui_workspace_bytes(const vui_config* cfg, int max_batch);
/* Bytes of ONE of the two (K or V) backbone caches: layers * slots * S * KV * hd elements.
 * Layout (layers, slots, S, KV, hd); layer l's (slots, S, KV, hd) slab is what the reference
 * calls flash_kv_caches[l].k_cache (model.py:71-99, 473-495). */
int64_t vui_kv_bytes(const vui_config* cfg);

/* Host-side object holding the configuration and the device pointers.  The workspace must
 * stay valid and must not be shared with another context that runs concurrently.
 * Stands in for Vui.setup_decode_graph's static buffers (model.py:1228-1246) and
 * RQTransformer.setup_cuda_graph_kv's (model.py:841-858). */
int vui_ctx_create(const vui_config* cfg, const vui_weights* w, void* workspace, int64_t workspace_bytes,
                   int max_batch, vui_ctx** out);
void vui_ctx_destroy(vui_ctx* ctx);
/* Device-side initialisation of the workspace (zeroes counters, exchange words and the error word, writes
 * the prefill copy of the projection weights: the weight tensors must hold their final values).  Enqueues
 * on stream AND waits for the stream before it returns (it copies from host locals and then asks the
 * runtime how many workgroups can be resident).  May be called again to clear a raised error word. */
int vui_ctx_init(vui_ctx* ctx, vui_stream_t stream);

/* The batch-1 bf16 calls below run as one persistent kernel ("fused") when the device can keep
 * one workgroup per compute unit resident and the dimensions fit; otherwise, and for B > 1, fp32
 * or int8 weights, as a sequence of kernels.  vui_ctx_fused(ctx, enable): enable = 1/0 switches the
 * fused form on/off, -1 only queries; returns 1 when the fused form will be used, else 0 (then
 * vui_last_error() says why it is unavailable).  The answer is about a whole frame (vui_frame_step,
 * vui_rq_generate).  A depth head whose keys and values for one frame do not both fit in a compute unit's
 * local memory keeps its keys in the workspace and is still fused; when even its values alone do not fit,
 * vui_backbone_step alone still takes the fused form, under the same switch.  No counterpart in the reference. */
int vui_ctx_fused(vui_ctx* ctx, int enable);
/* A stream whose kernels run on compute units [first_cu, first_cu + n_cus) only (hipExtStreamCreateWithCUMask),
 * and a context whose batch-1 one-launch kernel uses `nwg` workgroups instead of one per compute unit of the whole
 * GPU (160, 192, 224 or all of them): together they leave the other compute units to other work of the same process while a frame step runs
 * (a persistent kernel needs every one of its workgroups resident: on a stream of its own with n_cus >= nwg it
 * has them).  vui_ctx_workgroups is called after vui_ctx_init (which restores the full width); with nwg below
 * the full width the batched persistent kernels (2..16 rows) are switched off for the context.  The stream is
 * kept for the life of the process: there is no destroy call (on this ROCm release creating a masked stream after
 * one had been destroyed crashed, and so did a mask that is not one contiguous range).  A persistent kernel needs a
 * range whose size is a multiple of 32, so that every shader engine of every XCD keeps the same number of compute units
 * (workgroups are dealt evenly over the engines; with an uneven share one engine cannot hold its part of the grid).
 * No counterpart in the reference. */
int vui_cu_stream_create(int first_cu, int n_cus, vui_stream_t* out);
int vui_ctx_workgroups(vui_ctx* ctx, int nwg);

/* 1 when the depth head of 2..16 rows runs as one persistent kernel (bf16, enough resident workgroups, the
 * fused form switched on), else 0 and vui_last_error() says why.  No counterpart in the reference. */
int vui_ctx_rq_batch(vui_ctx* ctx);
/* 1 when the backbone step of 2..16 rows (vui_backbone_step, and through it vui_frame_step) runs as one persistent
 * kernel (bf16 activations, bf16 or int8 weights, dimensions in multiples of 64, enough resident workgroups, the fused
 * form switched on), else 0 and vui_last_error() says why; the kernel sequence runs then.  n_splits is not used by the
 * persistent form: it deals its workgroups to key ranges by the rows' cache lengths.  No counterpart in the reference. */
int vui_ctx_bb_batch(vui_ctx* ctx);
/* Synchronous health check (a blocking 16-byte device-to-host copy): VUI_EHIP if a persistent launch gave up
 * waiting for another workgroup, or if the 32-bit launch count of the context has wrapped (after 2^32 - 1
 * persistent launches; the launch that would wrap does nothing).  Either way nothing was committed by the
 * failing launch and the context stays unusable until vui_ctx_init is called again. */
int vui_ctx_status(vui_ctx* ctx);

/* Test aid: overwrites the context's launch-count word (waits for the device).  With 0xFFFFFFFF the next
 * persistent launch finds its count wrapped, raises the error word (value 2) and ends without waiting for
 * anything: the way to exercise the failure protocol without making a kernel wait.  No counterpart in the reference. */
int vui_debug_set_epoch(vui_ctx* ctx, uint32_t value);

/* Profiling aid: fused launches made after this call let four workgroups (`workgroup`, +1, +8, +131;
 * those beyond the grid do not exist) each write up to `cap` words (100 MHz clock << 8 | phase tag)
 * into their region of the device buffer buf: 4 regions of cap + 1 words, the last word of a region
 * receives the count in its low 32 bits and the launch's shader cycles above.  buf = NULL switches
 * it off.  No counterpart in the reference. */
int vui_debug_phase_clock(vui_ctx* ctx, uint64_t* buf, int cap, int workgroup);

/* One backbone decode step for B rows (B <= max_batch).
 *   Engine._backbone_decode_body / _backbone_decode_body_b  (engine.py:434-449, 485-502)
 *   Vui._decode_step_inner                                  (model.py:1280-1287)
 * Exactly one of codes_in / emb_in is non-NULL:
 *   codes_in  device (B, Q) int64: the previous frame, zero-padded to Q (engine.py:473-479)
 *   emb_in    device (B, d) dtype: a ready embedding (text/speaker token; prefill, engine.py:674-694)
 * slot_idx   device (B) int32 row -> KV slot, or NULL for the identity map
 * seq_lens   device (n_slots) int32: position at which each slot's new K/V row is written;
 *            after the step seq_lens[slot] += 1 for the B rows' slots (seq_inc == NULL), or
 *            seq_lens[s] += seq_inc[s] for every slot (engine.py:502)
 * k_cache/v_cache  device, layout above
 * hidden_out (B, d), cb0_out (B, CS), eos_out (B, 1): dtype, device; any may be NULL to skip
 * n_splits   key-range splits per (row, head) in attention, fixed per captured graph (>=1) */
int vui_backbone_step(vui_ctx* ctx, const int64_t* codes_in, const void* emb_in, const int32_t* slot_idx,
                      int32_t* seq_lens, const int32_t* seq_inc, int B, void* k_cache, void* v_cache,
                      void* hidden_out, void* cb0_out, void* eos_out, int n_splits, vui_stream_t stream);

/* Sampling parameters shared by the two samplers.  The uniform for (row b, codebook c) of
 * frame f is Philox4x32-10(key = seed, counter = (f, b, c, 0)); *frame_ctr is read on the
 * device, so a captured graph can be replayed with a new frame number. */
/* Sampling settings kept in DEVICE memory (16 bytes), read by the kernels when they run: a step recorded into a HIP
 * graph with vui_sample_params.dev set serves every temperature, top-k and seed - the host rewrites the block
 * (an ordinary stream-ordered copy) instead of capturing a graph per setting.  The reference keeps its temperature
 * in a 0-d device tensor filled before each replay for the same reason (model.py:1011). */
typedef struct vui_sample_dev {
  float temperature;
  int32_t top_k;
  uint64_t seed;
} vui_sample_dev;

typedef struct vui_sample_params {
  float temperature;      /* <= 0 means greedy */
  int32_t top_k;          /* 1 = greedy (lowest index of the maximum), <= 0 = no truncation */
  uint64_t seed;
  const int32_t* frame_ctr; /* device (1) int32 frame number, or NULL for frame 0 */
  const int32_t* state_rows; /* device (B) int32 or NULL: row b of a code-0 call uses the repetition state and the
                                random-stream row of state_rows[b] (continuous batching: the physical slot,
                                Engine._rep_apply_slots / _rep_push_slots, engine.py:594-616) */
  int32_t keep_ties;      /* code-0 sampler only.  0: Engine._sample_cb0's rule, exactly top_k probabilities kept
                             (topk + scatter, engine.py:855-863; ties at the k-th place go to the lowest indices).
                             1: sampling.sample_top_k's rule used by inference.stream_frames, everything >= the
                             k-th largest kept (sampling.py:14-20).  The depth head always keeps ties (model.py:955-962). */
  float top_p;            /* vui_sample_cb0 / vui_sample_logits only, 0 = off.  > 0: the nucleus cut of
                             sampling.sample_top_p (sampling.py:23-31) ahead of the top-k cut: in the order "largest
                             probability first" an entry is kept while the probability strictly ahead of it is
                             <= top_p.  With top_k > 0 this is sample_top_p_top_k (sampling.py:34-43): of the
                             nucleus, everything >= its k-th largest entry.  Equal probabilities are ordered by
                             index (torch.sort leaves that open).  The other entry points require 0. */
  const vui_sample_dev* dev; /* device pointer or NULL.  Set: temperature, top_k and seed are read from there on
                                the device at run time and the three fields above are ignored. */
} vui_sample_params;

/* Device-side end-of-turn test of a streamed turn (Engine._stream_row's `step >= min_frames and sigmoid(eos) >
 * eos_threshold`, engine.py:1468-1471) so that the host need not wait for every frame before it enqueues the next.
 * state: device int32[2] = {stopped, step}; the host writes {0, 1} when a chunk's first frame has been drawn.
 * A frame step given this struct (batch 1 only) does nothing at all while stopped != 0; otherwise it runs, then sets
 * stopped = 1 if step >= min_frames and its EOS probability exceeds threshold, and increments step.  The step that
 * sets the flag is the reference's last one (a step whose persistent launch failed sets it to 2 instead): its frame is to be dropped by the caller, its position and repetition
 * push stay.  Only the one-launch form skips stopped steps; the kernel-sequence form maintains the flag but runs
 * every step it is given (vui_ctx_fused tells which form a context uses), so there the caller reads the flag
 * before it enqueues the next step.  No counterpart in the reference (its loop reads the logit with .item()). */
typedef struct vui_eos_stop {
  float threshold;
  int32_t min_frames;
  int32_t* state;
} vui_eos_stop;

/* Code-0 sampler with repetition penalty for B rows:
 *   Engine._rep_apply / _sample_cb0 / _rep_push  (engine.py:571-590, 855-863, 1451-1466)
 * logits (B, CS) dtype device; rep_counts (B, CS) fp32 device or NULL; rep_hist (B, window)
 * int32 and rep_pos (B, 2) int32 {head, filled} device ring state or NULL (no window);
 * code0_out (B) int64 device. */
int vui_sample_cb0(vui_ctx* ctx, const void* logits, float* rep_counts, int32_t* rep_hist, int32_t* rep_pos,
                   float penalty, int window, const vui_sample_params* sp, int64_t* code0_out, int B,
                   vui_stream_t stream);

/* RQ depth head: all remaining codebooks of one frame for B rows.
 *   RQTransformer._generate_graph_body_kv / generate_cuda_graph_kv  (model.py:908-1016)
 * hidden (B, d) dtype, code0 (B) int64, logit_bias (Q-1, CS) fp32 or NULL, n_q = Q' in [2, Q];
 * codes_out (B, codes_stride) int64: columns [0, Q') written, columns [Q', codes_stride)
 * zeroed when zero_pad != 0 (the padding the next backbone step expects). */
int vui_rq_generate(vui_ctx* ctx, const void* hidden, const int64_t* code0, const float* logit_bias,
                    int n_q, const vui_sample_params* sp, int64_t* codes_out, int codes_stride, int zero_pad,
                    int B, vui_stream_t stream);

/* Prompt ingestion: T new positions of ONE row in one pass per layer (GEMMs on the matrix cores,
 * causal attention against the cache), bf16 weights only.
 *   Decoder.forward_flash with T > 1 / Engine._prefill_emb  (model.py:534-549, engine.py:674-694)
 * emb_in (T, d) bf16 device: the embeddings to append at positions pos0 .. pos0+T-1 of `slot`
 * (pos0 is the slot's current length, passed from the host because the launch shapes depend on it);
 * K/V rows are appended to the caches, seq_lens[slot] becomes pos0 + T, hidden_out (T, d) bf16
 * receives the final-norm outputs.  scratch: device memory of vui_prefill_scratch_bytes(cfg, T,
 * pos0 + T) bytes, 256-byte aligned; the library allocates nothing.  vui_prefill_scratch_bytes returns
 * VUI_EINVAL for a configuration the pass does not take (fp32 or int8 weights, d_model / heads x head_dim /
 * ffn not multiples of 64, head_dim not a multiple of 32): such prompts go position by position through
 * vui_backbone_step.  Calls for different slots may be in flight on different streams at once if each has a
 * scratch buffer of its own: beyond the caller's buffers a call touches only read-only weights. */
int64_t vui_prefill_scratch_bytes(const vui_config* cfg, int T, int L);
int vui_prefill(vui_ctx* ctx, const void* emb_in, int T, int slot, int pos0, int32_t* seq_lens, void* k_cache,
                void* v_cache, void* hidden_out, void* scratch, int64_t scratch_bytes, vui_stream_t stream);

/* The whole per-frame step: backbone step on codes_io, code-0 sampling, RQ head; the new frame
 * is written back to codes_io (zero-padded to Q) so the call can be repeated or replayed.
 *   Engine._stream_row / _render_rows loop body (engine.py:1450-1485, 1011-1044)
 * frames_out: optional device (max_frames, B, Q) int64 log; the frame goes to row *frame_ctr.
 * eos_prob_out fp32 device, may be NULL: sigmoid(eos logit) (engine.py:1468-1471); (B) values, or,
 *   when frames_out is given, a (max_frames, B) log whose row *frame_ctr is written.  A batch-1 step whose
 *   persistent launch failed (see vui_ctx_status) writes -1 there and commits nothing else.
 * frame_ctr (device int32) is incremented at the end of the step.
 * stop: NULL, or the device-side end-of-turn test described at vui_eos_stop (B == 1). */
int vui_frame_step(vui_ctx* ctx, int64_t* codes_io, const int32_t* slot_idx, int32_t* seq_lens,
                   const int32_t* seq_inc, int B, void* k_cache, void* v_cache, float* rep_counts,
                   int32_t* rep_hist, int32_t* rep_pos, float penalty, int window,
                   const vui_sample_params* sp_cb0, const vui_sample_params* sp_rq, const float* logit_bias,
                   int n_q, void* hidden_out, void* cb0_out, float* eos_prob_out, int64_t* frames_out,
                   int max_frames, int32_t* frame_ctr, int n_splits, const vui_eos_stop* stop, vui_stream_t stream);

/* HIP graph helpers (stand in for torch.cuda.CUDAGraph capture/replay, model.py:873-876,
 * 1254-1256; engine.py:465-468).  begin/end bracket any sequence of the calls above issued
 * on `stream`; the returned handle is replayed with vui_graph_launch. */
typedef struct vui_graph vui_graph;
int vui_graph_begin(vui_stream_t stream);
int vui_graph_end(vui_stream_t stream, vui_graph** out);
int vui_graph_launch(vui_graph* g, vui_stream_t stream);
void vui_graph_destroy(vui_graph* g);

/* ---- single kernels, for micro-benchmarks and unit parity tests ---- */

/* y = [rmsnorm_w(x)] W^T for B rows.  x (B, K), W (N, K), y (B, N); norm_w (K) or NULL.
 * RMSNorm.forward + nn.Linear (model.py:286-297, 158, 220).  w_int8 != 0: W is int8 with
 * `scales` (N) dtype. */
int vui_rmsnorm_gemv(int dtype, const void* x, const void* norm_w, float eps, const void* W, const void* scales,
                     int w_int8, void* y, int B, int N, int K, vui_stream_t stream);
/* In-place interleaved rotation of x (B, n_heads, head_dim) at positions pos (B) int32.
 * apply_rotary_emb (rope.py:23-57). */
int vui_rope(int dtype, void* x, const float* rope_table, const int32_t* pos, int B, int n_heads, int head_dim,
             int rope_dim, vui_stream_t stream);
/* Decode attention for B rows over caches (slots, S, KV, hd): appends k_new/v_new (B, KV, hd)
 * at seq_lens[slot] (when non-NULL), then out (B, H, hd) = softmax(q K^T / sqrt(hd)) V over
 * positions 0..seq_lens[slot].  flash_attn_with_kvcache (model.py:247-257).
 * scratch: device, vui_attn_scratch_bytes(B, H, hd, n_splits) bytes, zero-initialised once. */
int64_t vui_attn_scratch_bytes(int B, int H, int hd, int n_splits);
int vui_decode_attn(int dtype, const void* q, const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                    const int32_t* seq_lens, const int32_t* slot_idx, void* out, int B, int H, int KV, int hd,
                    int S, int window, int n_splits, void* scratch, vui_stream_t stream);
/* vui_decode_attn for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments without `scratch`, same kernels, same results.  It has
 * no counterpart in the reference.  The pieces of the key-range splits and their arrival counters live in a
 * fixed array inside the library's code object (4 MiB + 8 KiB per GPU, held until the process ends), so
 * B * H <= 2048 and B * H * n_splits * (hd + 2) * 4 <= 4 MiB; anything larger returns VUI_EINVAL and belongs to
 * vui_decode_attn.  The call allocates and frees nothing (the array's address is looked up once per device, at
 * vui_ctx_init or on the first call there, so make one of those before a graph capture); the counters are
 * cleared by a small fill kernel at the start of every call.  All calls on one GPU share the one array: calls
 * that overlap there (two streams, two threads, two replays in flight) race; serialise them. */
int vui_decode_attn_noalloc(int dtype, const void* q, const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                            const int32_t* seq_lens, const int32_t* slot_idx, void* out, int B, int H, int KV, int hd,
                            int S, int window, int n_splits, vui_stream_t stream);
/* One draw per row from logits (B, CS) fp32 with the RQ-head rule (model.py:955-962). */
int vui_sample_logits(const float* logits, const float* bias, int CS, const vui_sample_params* sp, int codebook,
                      int64_t* out, int B, vui_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* VUI_AMD_H */
