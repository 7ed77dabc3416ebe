// Internal launcher interface between the kernel translation units and the C ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/vui_amd.h"

// epilogues of the fused GEMV
enum {
  EPI_STORE = 0,   // y = rnd(acc)
  EPI_RESID = 1,   // y = rnd(resid + rnd(acc))
  EPI_SWIGLU = 2,  // y = rnd(rnd(silu(rnd(acc1))) * rnd(acc3))   (two weight matrices)
  EPI_QKV = 3,     // split into q | k | v, rotate q and k, append k and v to the KV cache
  EPI_ADDVEC = 4,  // y = rnd(rnd(acc) + vec[n])
  EPI_RQ_QKV = 5,  // split into q | k | v without rotation, k/v into the depth-head cache
};

// per-layer attention window and rotation table (global-attention layers, vui_config.global_layers)
static inline bool layer_is_global(const vui_config& c, int l) { return (c.global_layers >> l) & 1ull; }
static inline int layer_window(const vui_config& c, int l) { return layer_is_global(c, l) ? 0 : c.window; }
static inline const float* layer_rope(const vui_config& c, const vui_weights& w, int l, int* rope_dim) {
  if (layer_is_global(c, l) && w.rope_table_global) { *rope_dim = c.global_rope_dim; return w.rope_table_global; }
  *rope_dim = c.rope_dim;
  return w.rope_table;
}

struct GemvArgs {
  int dtype;      // VUI_DTYPE_*
  int w_int8;     // weights are int8 with per-row scales
  const void* x;  // (B, K)
  const void* norm_w;  // (K) or nullptr: no RMSNorm prologue
  float eps;
  const void* W;   // (N, K)
  const void* W2;  // second matrix for EPI_SWIGLU
  const void* sc;  // (N) scales for int8
  const void* sc2;
  void* y;         // (B, ldy)
  int ldy;
  const void* resid;  // (B, ldy) for EPI_RESID (may alias y)
  const void* vec;    // (N) for EPI_ADDVEC
  int B, N, K;
  int epi;
  // EPI_QKV / EPI_RQ_QKV
  const float* rope;  // (S, rope_dim, 2)
  int rope_dim, hd, nq, nkv;  // nq = H*hd, nkv = KV*hd
  void* kc;           // layer slab (slots, S, KV, hd)  | depth-head (B, Q, R)
  void* vc;
  const int32_t* seq_lens;
  const int32_t* slot_idx;
  int S;       // cache length (positions)
  int rq_pos;  // EPI_RQ_QKV: position written
  // optional extra output row with bias (the eos head), plus the position update it carries
  const void* Wx;  // (1, K)
  const void* bx;  // (1)
  void* yx;        // (B, 1)
  void* hid_out;   // (B, K): the staged (normalised) activations, written by the extra block
  int32_t* upd_seq_lens;       // if set: after the step seq_lens are advanced by the extra block
  const int32_t* upd_seq_inc;  // (n_slots) or nullptr (+1 for the B rows' slots)
  int n_slots;
};

int launch_gemv(const GemvArgs& a, hipStream_t st);
// 16-row MFMA form of the same operation (gemm16.hip); the extra row / position update of `a` is not handled there
bool gemm16_supported(const GemvArgs& a);
int launch_gemm16(const GemvArgs& a, hipStream_t st);

struct AttnArgs {
  int dtype;
  const void* q;  // (B, H*hd), already rotated
  const void* kc; // (slots, S, KV, hd) with the new row already appended
  const void* vc;
  const int32_t* seq_lens;  // position of the newest key per slot
  const int32_t* slot_idx;
  void* out;  // (B, H*hd)
  int B, H, KV, hd, S, window, n_splits;
  float* part;        // (B, H, n_splits, hd + 2) fp32
  uint32_t* counter;  // (B*H), zero between launches
};
int launch_decode_attn(const AttnArgs& a, hipStream_t st);
int launch_kv_append(int dtype, const void* k_new, const void* v_new, void* kc, void* vc, const int32_t* seq_lens,
                     const int32_t* slot_idx, int B, int KV, int hd, int S, hipStream_t st);

int launch_embed(int dtype, const int64_t* codes, const void* table, void* x, int B, int Q, int CS, int d,
                 hipStream_t st);
int launch_copy_rows(int dtype, const void* src, void* dst, int64_t n, hipStream_t st);
int launch_rope(int dtype, void* x, const float* table, const int32_t* pos, int B, int nh, int hd, int rope_dim,
                hipStream_t st);

struct RqAttnArgs {
  int dtype;
  const void* q;   // (B, R)
  const void* kc;  // (B, Q, R)
  const void* vc;
  void* out;  // (B, R)
  int B, heads, hd, Q, pos;
};
int launch_rq_attn(const RqAttnArgs& a, hipStream_t st);

struct SampleArgs {
  int dtype;           // element type of logits (VUI_DTYPE_F32 allowed for the raw entry point)
  const void* logits;  // (B, CS)
  const float* bias;   // (CS) fp32 or nullptr
  float* rep_counts;   // (B, CS) or nullptr
  int32_t* rep_hist;   // (B, window) or nullptr
  int32_t* rep_pos;    // (B, 2) {head, filled}
  float penalty;
  int window;
  float temperature;
  int top_k;
  float top_p;         // > 0: nucleus cut ahead of the top-k cut (stand-alone sampling kernel only)
  const vui_sample_dev* dev;  // if set: temperature, top_k, seed come from this device block
  uint64_t seed;
  const int32_t* frame_ctr;
  const int32_t* state_rows;  // (B) or nullptr: repetition state / random-stream row of row b
  int codebook;  // Philox counter word 2
  int exact_k;   // code-0 rule: exactly top_k entries kept, ties at the k-th place cut in index order
  int CS, B;
  int64_t* out;  // out[b * out_stride + out_col]
  int out_stride, out_col;
  // optional: build the depth head's next input token  x[b] = rnd(emb[code + emb_off] + pos_vec)
  const void* tok_emb;  // (rows, R)
  const void* tok_pos;  // (R)
  void* tok_out;        // (B, R)
  int64_t tok_emb_off;
  int R;
  // optional: eos probability = sigmoid(eos_logit[b])
  const void* eos_logit;  // (B) dtype
  float* eos_prob;        // (B)
  // optional zero padding of out[b, pad_from..pad_to)
  int pad_from, pad_to;
};
int launch_sample(const SampleArgs& a, hipStream_t st);

// x[b] = rnd(emb[code[b] + off] + pos_vec); optionally codes_out[b*stride] = code[b]
int launch_rq_token(int dtype, const int64_t* code, int64_t off, const void* emb, const void* pos_vec, void* x,
                    int B, int R, int64_t* codes_out, int stride, int CS, hipStream_t st);
// frames_out[*ctr] = codes (B*Q) if ctr < max_frames; *ctr += 1
// and eos_out[(frames_out ? *ctr : 0) * B + b] = eos_in[b]
int launch_frame_finish(const int64_t* codes, int64_t* frames_out, int n, int max_frames, int32_t* ctr,
                        const float* eos_in, float* eos_out, int B, int32_t* stop_state, float stop_thr, int stop_min,
                        hipStream_t st);
int launch_add_rows(int dtype, const void* a, const void* vec, void* out, int B, int R, hipStream_t st);
int launch_fill_u32(uint32_t* p, uint32_t v, int64_t n, hipStream_t st);

// ---- fused frame kernel (frame.hip) ----
struct FrameArgs {
  int d, L, H, KV, hd, F, Q, CS, R, rqL, rqH, rqF, rope_dim, S, window;
  float eps, rq_eps;
  const vui_weights* w;  // device copy
  // backbone
  const int64_t* codes_in;
  const uint16_t* emb_in;
  const int32_t* slot_idx;
  int32_t* seq_lens;
  const int32_t* seq_inc;
  int n_slots;
  unsigned long long global_layers;  // bit l: layer l attends over the whole cache and uses the global rotation table
  int global_rope_dim;
  uint16_t *kc, *vc;
  uint16_t *hidden_out, *cb0_out, *eos_out;
  // code-0 sampling
  float* rep_counts;
  int32_t* rep_hist;
  int32_t* rep_pos;
  float penalty;
  int rep_window;
  float temp0; int topk0;
  float temp1; int topk1;
  uint64_t seed0, seed1;
  const vui_sample_dev *sdev0, *sdev1;  // if set: the settings of the code-0 draw / the depth head's draws, read on the device
  const int32_t* frame_ctr0;
  const int32_t* frame_ctr1;
  int64_t* code0_out;
  // depth head
  const uint16_t* rq_hidden;
  const int64_t* rq_code0;
  const float* logit_bias;
  int n_q;
  int64_t* codes_out;
  int codes_stride, zero_pad;
  // frame bookkeeping
  int64_t* frames_out;
  float* eos_prob_out;
  int max_frames;
  int32_t* frame_ctr;
  int32_t* stop_state;  // {stopped, step} or nullptr (vui_eos_stop)
  float stop_thr;
  int stop_min;
  int exact0;           // code-0 cut keeps exactly top_k entries
  // exchange
  uint64_t* ll;
  uint32_t* epoch;
  uint32_t* arrive;
  uint32_t* err;
  int ns;    // attention key splits per head
  int mode;  // FR_* bits
  int lds_kv_off;  // byte offset of the depth-head K/V store in LDS
  int w_int8;      // 1: the backbone's matrices are int8 with per-row scales
  int rq_kg;       // 1: depth-head keys in rq_kscratch (a region per workgroup), values in LDS
  uint16_t* rq_kscratch;
  uint64_t* prof;  // optional (prof_cap + 1) words: (clock << 8 | tag) per phase point, count in the last word
  int prof_cap, prof_wg;
  int lds_prof_off;  // set by launch_frame: LDS offset of the stamp buffer
};

enum { FR_BACKBONE = 1, FR_CB0 = 2, FR_RQ = 4, FR_FINISH = 8 };

size_t frame_ll_words(const vui_config& c, int ns);
size_t frame_lds_bytes(const vui_config& c);
size_t frame_rq_cache_bytes(const vui_config& c);
size_t frame_rq_lds_cache_bytes(const vui_config& c);
int frame_rq_keys_global(const vui_config& c);
size_t frame_rq_key_scratch_bytes(const vui_config& c, int nwg);
size_t frame_lds_bytes_backbone(const vui_config& c);
bool frame_supported(const vui_config& c, int nwg, int ns, bool with_rq, char* why, size_t why_len);
int frame_max_resident(size_t lds_bytes, int* n_cu);
int launch_frame(const FrameArgs& a, int nwg, size_t lds_bytes, hipStream_t st);

// rqbatch.hip
size_t rq_batch_ll_words(const vui_config& c);
size_t rq_batch_lds_bytes(const vui_config& c);
bool rq_batch_supported(const vui_config& c, int nwg, char* why, size_t why_len);
size_t rq_batch_weight_bytes(const vui_config& c, int nwg);  // tiled copies of the depth head's matrices; 0: kernel unavailable
int rq_batch_tile_weights(const vui_config& c, const vui_weights& w, void* dst, vui_weights* tiled, hipStream_t st);
int rq_batch_max_resident(size_t lds_bytes);
int launch_rq_batch(const vui_config& c, const vui_weights* wdev, const void* hidden, const int64_t* code0, const float* logit_bias,
                    int n_q, float temp, int topk, uint64_t seed, const vui_sample_dev* sdev, const int32_t* frame_ctr, int64_t* codes_out,
                    int codes_stride, int zero_pad, int B, uint64_t* ll, uint32_t* ctl, int nwg, hipStream_t st);

// bbatch.hip: the backbone step of 2..16 rows as one persistent kernel
bool bb_batch_supported(const vui_config& c, int nwg, char* why, size_t why_len);
size_t bb_batch_ll_words(const vui_config& c, int nwg);
size_t bb_batch_lds_bytes(const vui_config& c);
size_t bb_batch_weight_bytes(const vui_config& c, int nwg);   // own tiled copy of the layers' matrices (int8 contexts; bf16 ones without the prefill copy), else 0
size_t bb_batch_head_bytes(const vui_config& c, int nwg);     // tiled copy of the codec head
int bb_batch_tile_weights(const vui_config& c, const vui_weights& w, void* dst_layers, void* dst_head, hipStream_t st);
int bb_batch_max_resident(const vui_config& c);
int launch_bb_batch(const vui_config& c, const vui_weights* wdev, const void* tiled_layers, const void* tiled_head, const int64_t* codes_in,
                    const void* emb_in, const int32_t* slot_idx, int32_t* seq_lens, const int32_t* seq_inc, int B, void* k_cache,
                    void* v_cache, void* hidden_out, void* cb0_out, void* eos_out, uint64_t* ll, uint32_t* ctl, int nwg, hipStream_t st);

// prefill.hip
size_t prefill_scratch_bytes(const vui_config& c, int T, int L);
bool prefill_supported(const vui_config& c, char* why, size_t why_len);
size_t prefill_weight_bytes(const vui_config& c);  // the projection weights in the GEMMs' operand layout; 0: no pass
int prefill_tile_weights(const vui_config& c, const vui_weights& w, void* dst, hipStream_t st);
int launch_prefill(const vui_config& c, const vui_weights& w, const void* tiled_w, const void* emb, int T, int slot, int pos0,
                   int32_t* seq_lens, void* k_cache, void* v_cache, void* out, void* scratch, size_t scratch_bytes, hipStream_t st);

void vui_set_error(const char* fmt, ...);
#define HIP_TRY(expr)                                                                  \
  do {                                                                                 \
    hipError_t _e = (expr);                                                            \
    if (_e != hipSuccess) {                                                            \
      vui_set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
      return VUI_EHIP;                                                                 \
    }                                                                                  \
  } while (0)
