// C ABI: context, per-step kernel sequences, HIP graph helpers.  See include/vui_amd.h.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <new>

#include "internal.h"
#include <hip/hip_ext.h>

static thread_local char g_err[512] = "";

void vui_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

#define MAX_SPLITS 64

// ---- scratch of the entry point that allocates nothing (vui_decode_attn_noalloc) ----
// One array per GPU, part of the code object: [arrival counters: NOALLOC_MAX_ROWS_HEADS words][pieces].  In host
// code the array's name stands for the symbol, not for device memory: its address on the current device comes
// from hipGetSymbolAddress, once per device, and only that pointer is handed to kernels.
#define NOALLOC_MAX_ROWS_HEADS 2048
#define NOALLOC_PIECE_BYTES (4 << 20)
#define NOALLOC_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[NOALLOC_MAX_ROWS_HEADS * 4 + NOALLOC_PIECE_BYTES];
static std::mutex g_noalloc_mu;
static unsigned char* g_noalloc_ptr[NOALLOC_MAX_DEVICES];

static int noalloc_scratch(unsigned char** out) {
  int dev = -1;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) { vui_set_error("device ordinal %d outside [0, %d)", dev, NOALLOC_MAX_DEVICES); return VUI_EINVAL; }
  std::lock_guard<std::mutex> lock(g_noalloc_mu);
  if (!g_noalloc_ptr[dev]) {
    void* p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) { vui_set_error("hipGetSymbolAddress returned no address for the built-in scratch"); return VUI_EHIP; }
    g_noalloc_ptr[dev] = (unsigned char*)p;
  }
  *out = g_noalloc_ptr[dev];
  return VUI_OK;
}

struct vui_ctx {
  vui_config cfg;
  vui_weights w;
  int max_batch;
  size_t esz;
  // workspace carve-up
  char* base;
  void *x, *q, *att, *h, *hidden, *cb0, *eos;
  float* part;
  uint32_t* counter;
  void *rx, *rq_q, *rq_att, *rq_h, *rq_kc, *rq_vc, *rq_logits;
  int64_t* code0;
  float* eos_prob;
  // fused frame kernel
  uint64_t* ll;
  size_t ll_words;
  vui_weights* wdev;
  uint32_t* ctl;  // [0] epoch, [1] arrive, [2] err
  void* pf_w;     // projection weights of every layer in the prefill GEMMs' operand layout (bf16 contexts)
  void* rq_tw;    // the depth head's matrices in the batched kernel's operand layout
  vui_weights* wdev_t;  // device copy of the weight table with those matrices' pointers
  void* rq_ks;          // depth-head keys of the one-launch kernel when they do not fit in LDS (a region per workgroup)
  int fused_ok, fused_on, nwg, ns;
  int fused_bb_ok;      // the backbone step alone can run as the one-launch kernel (its LDS need is smaller)
  size_t lds_bytes, lds_bb;
  char fused_why[96];
  uint64_t* prof;
  int prof_cap, prof_wg;
  // persistent depth head for 2..16 rows
  int rqb_ok;
  char rqb_why[96];
  // persistent backbone step for 2..16 rows
  int bb_ok;
  char bb_why[96];
  void* bb_w8;    // the layers' matrices in the kernel's operand layout where it keeps a copy of its own (int8; bf16 without the prefill copy)
  size_t bb_w8_bytes;
  void* bb_head;  // the codec head in that layout
};

#define FUSED_NWG 256
#define FUSED_NS 32

// the batch-1 frame kernel and the batched depth head never run at the same time: one exchange area
static size_t ll_words_needed(const vui_config& c) {
  const size_t a = frame_ll_words(c, FUSED_NS), b = (c.dtype == VUI_DTYPE_BF16 && c.rq_layers > 0) ? rq_batch_ll_words(c) : 0;
  const size_t e = bb_batch_supported(c, FUSED_NWG, nullptr, 0) ? bb_batch_ll_words(c, FUSED_NWG) : 0;
  const size_t m = a > b ? a : b;
  return m > e ? m : e;
}

struct Carve {
  size_t off = 0;
  size_t take(size_t bytes) {
    size_t o = off;
    off += (bytes + 255) & ~(size_t)255;
    return o;
  }
};

static int check_cfg(const vui_config* c, int max_batch) {
  if (!c) { vui_set_error("config is NULL"); return VUI_EINVAL; }
  if (c->dtype != VUI_DTYPE_BF16 && c->dtype != VUI_DTYPE_F32) { vui_set_error("bad dtype %d", c->dtype); return VUI_EINVAL; }
  if (max_batch < 1 || max_batch > VUI_MAX_BATCH) { vui_set_error("max_batch %d out of [1,%d]", max_batch, VUI_MAX_BATCH); return VUI_EINVAL; }
  if (c->n_layers < 1 || c->n_layers > VUI_MAX_LAYERS || c->rq_layers < 0 || c->rq_layers > VUI_MAX_RQ_LAYERS) {
    vui_set_error("layer counts out of range (%d, %d)", c->n_layers, c->rq_layers); return VUI_EINVAL; }
  if (c->n_heads < 1 || c->n_kv_heads < 1 || c->n_heads % c->n_kv_heads || c->n_heads * c->head_dim != c->d_model) {
    vui_set_error("bad head layout H=%d KV=%d hd=%d d=%d", c->n_heads, c->n_kv_heads, c->head_dim, c->d_model); return VUI_EINVAL; }
  if ((c->head_dim & 7) || c->head_dim > 128 || (c->d_model & 7) || (c->ffn & 7)) {
    vui_set_error("head_dim (<=128), d_model and ffn must be multiples of 8"); return VUI_EINVAL; }
  if (c->rope_dim < 0 || c->rope_dim > c->head_dim || (c->rope_dim & 1)) { vui_set_error("bad rope_dim %d", c->rope_dim); return VUI_EINVAL; }
  if (c->n_quantizers < 2 || c->n_quantizers > 64 || c->codebook_size < 2 || c->codebook_size > 8192) {
    vui_set_error("n_quantizers in [2,64], codebook_size in [2,8192] required"); return VUI_EINVAL; }
  if (c->rq_layers > 0 && (c->rq_heads < 1 || c->rq_dim < 8 || c->rq_dim % c->rq_heads || (c->rq_dim & 7) || (c->rq_ffn & 7) ||
                           c->rq_dim / c->rq_heads > 128)) {
    vui_set_error("bad depth-head layout R=%d heads=%d ffn=%d", c->rq_dim, c->rq_heads, c->rq_ffn); return VUI_EINVAL; }
  if (c->max_seqlen < 1 || c->n_slots < 1) { vui_set_error("max_seqlen and n_slots must be positive"); return VUI_EINVAL; }
  if (c->int8_backbone && c->dtype != VUI_DTYPE_BF16) { vui_set_error("int8 weights need bf16 activations"); return VUI_EINVAL; }
  if (c->global_rope_dim < 0 || c->global_rope_dim > c->head_dim || (c->global_rope_dim & 1)) { vui_set_error("bad global_rope_dim %d", c->global_rope_dim); return VUI_EINVAL; }
  if (c->n_layers < 64 && (c->global_layers >> c->n_layers)) { vui_set_error("global_layers names layers beyond n_layers"); return VUI_EINVAL; }
  return VUI_OK;
}

static size_t carve(const vui_config* c, int Bm, vui_ctx* x) {
  const size_t e = c->dtype == VUI_DTYPE_F32 ? 4 : 2;
  const size_t d = c->d_model, R = c->rq_dim;
  Carve cv;
  size_t o;
#define TAKE(field, type, bytes) o = cv.take(bytes); if (x) x->field = (type)(x->base + o)
  TAKE(x, void*, Bm * d * e);
  TAKE(q, void*, Bm * d * e);
  TAKE(att, void*, Bm * d * e);
  TAKE(h, void*, (size_t)Bm * c->ffn * e);
  TAKE(hidden, void*, Bm * d * e);
  TAKE(cb0, void*, (size_t)Bm * c->codebook_size * e);
  TAKE(eos, void*, Bm * e);
  TAKE(part, float*, (size_t)Bm * c->n_heads * MAX_SPLITS * (c->head_dim + 2) * 4);
  TAKE(counter, uint32_t*, (size_t)Bm * c->n_heads * 4);
  TAKE(rx, void*, Bm * R * e);
  TAKE(rq_q, void*, Bm * R * e);
  TAKE(rq_att, void*, Bm * R * e);
  TAKE(rq_h, void*, (size_t)Bm * c->rq_ffn * e);
  TAKE(rq_kc, void*, (size_t)c->rq_layers * Bm * c->n_quantizers * R * e);
  TAKE(rq_vc, void*, (size_t)c->rq_layers * Bm * c->n_quantizers * R * e);
  TAKE(rq_logits, void*, (size_t)Bm * c->codebook_size * e);
  TAKE(code0, int64_t*, Bm * 8);
  TAKE(eos_prob, float*, Bm * 4);
  TAKE(ll, uint64_t*, ll_words_needed(*c) * 8);
  TAKE(wdev, vui_weights*, sizeof(vui_weights));
  TAKE(ctl, uint32_t*, 256);
  TAKE(pf_w, void*, prefill_weight_bytes(*c));  // empty when the configuration has no prefill pass
  TAKE(rq_tw, void*, rq_batch_weight_bytes(*c, FUSED_NWG));  // empty when the batched depth-head kernel is unavailable
  TAKE(wdev_t, vui_weights*, sizeof(vui_weights));
  TAKE(rq_ks, void*, frame_rq_key_scratch_bytes(*c, FUSED_NWG));
  TAKE(bb_w8, void*, bb_batch_weight_bytes(*c, FUSED_NWG));  // empty for bf16 weights with a prefill copy (that one serves) or when the kernel is unavailable
  TAKE(bb_head, void*, bb_batch_head_bytes(*c, FUSED_NWG));
#undef TAKE
  return cv.off;
}

extern "C" {

const char* vui_last_error(void) { return g_err; }
int vui_version(void) { return 1; }

int64_t vui_workspace_bytes(const vui_config* cfg, int max_batch) {
  if (check_cfg(cfg, max_batch)) return VUI_EINVAL;
  return (int64_t)carve(cfg, max_batch, nullptr);
}

int64_t vui_kv_bytes(const vui_config* c) {
  if (!c) return VUI_EINVAL;
  return (int64_t)c->n_layers * c->n_slots * c->max_seqlen * c->n_kv_heads * c->head_dim * (c->dtype == VUI_DTYPE_F32 ? 4 : 2);
}

int vui_ctx_create(const vui_config* cfg, const vui_weights* w, void* workspace, int64_t workspace_bytes, int max_batch,
                   vui_ctx** out) {
  if (!out || !w || !workspace) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  int rc = check_cfg(cfg, max_batch);
  if (rc) return rc;
  const size_t need = carve(cfg, max_batch, nullptr);
  if ((size_t)workspace_bytes < need) { vui_set_error("workspace too small: %lld < %zu", (long long)workspace_bytes, need); return VUI_ENOMEM; }
  if (((uintptr_t)workspace) & 255) { vui_set_error("workspace must be 256-byte aligned"); return VUI_EINVAL; }
  if (!w->audio_emb || !w->final_norm || !w->codec_head || !w->eos_w || !w->eos_b || (cfg->rope_dim && !w->rope_table)) {
    vui_set_error("missing backbone weight pointer"); return VUI_EINVAL; }
  if (w->rope_table_global && cfg->global_rope_dim < 2) { vui_set_error("rope_table_global needs global_rope_dim >= 2"); return VUI_EINVAL; }
  for (int l = 0; l < cfg->n_layers; ++l) {
    const vui_layer_weights& L = w->layers[l];
    if (!L.attn_norm || !L.wqkv || !L.wo || !L.mlp_norm || !L.w1 || !L.w3 || !L.w2) { vui_set_error("missing weights of layer %d", l); return VUI_EINVAL; }
    if (cfg->int8_backbone && (!L.s_qkv || !L.s_o || !L.s_1 || !L.s_3 || !L.s_2)) { vui_set_error("missing int8 scales of layer %d", l); return VUI_EINVAL; }
  }
  if (cfg->rq_layers > 0) {
    if (!w->rq_code_emb || !w->rq_pos_emb || !w->rq_head_w || !w->rq_norm || (cfg->rq_dim != cfg->d_model && !w->rq_backbone_proj)) {
      vui_set_error("missing depth-head weight pointer"); return VUI_EINVAL; }
    for (int l = 0; l < cfg->rq_layers; ++l) {
      const vui_rq_layer_weights& L = w->rq_layers[l];
      if (!L.attn_norm || !L.wqkv || !L.wo || !L.mlp_norm || !L.w1 || !L.w3 || !L.w2) { vui_set_error("missing weights of depth-head layer %d", l); return VUI_EINVAL; }
    }
  }
  vui_ctx* c = new (std::nothrow) vui_ctx();
  if (!c) { vui_set_error("out of host memory"); return VUI_ENOMEM; }
  c->cfg = *cfg;
  c->w = *w;
  c->max_batch = max_batch;
  c->esz = cfg->dtype == VUI_DTYPE_F32 ? 4 : 2;
  c->base = (char*)workspace;
  c->fused_ok = 0; c->fused_on = 1; c->fused_why[0] = 0;
  c->prof = nullptr; c->prof_cap = 0; c->prof_wg = 0;
  carve(cfg, max_batch, c);
  *out = c;
  return VUI_OK;
}

void vui_ctx_destroy(vui_ctx* ctx) { delete ctx; }

int vui_ctx_init(vui_ctx* ctx, vui_stream_t stream) {
  if (!ctx) { vui_set_error("NULL context"); return VUI_EINVAL; }
  hipStream_t st = (hipStream_t)stream;
  unsigned char* builtin = nullptr;
  int rc = noalloc_scratch(&builtin);  // the built-in scratch's address on this device, so that no later call has to ask
  if (rc) return rc;
  if ((rc = launch_fill_u32(ctx->counter, 0u, (int64_t)ctx->max_batch * ctx->cfg.n_heads, st))) return rc;
  // fused frame kernel: exchange words and control words start at zero (epoch 0 = "never written")
  ctx->ll_words = ll_words_needed(ctx->cfg);
  if ((rc = launch_fill_u32((uint32_t*)ctx->ll, 0u, (int64_t)ctx->ll_words * 2, st))) return rc;
  if ((rc = launch_fill_u32(ctx->ctl, 0u, 64, st))) return rc;
  HIP_TRY(hipMemcpyAsync(ctx->wdev, &ctx->w, sizeof(vui_weights), hipMemcpyHostToDevice, st));
  if (prefill_weight_bytes(ctx->cfg) && (rc = prefill_tile_weights(ctx->cfg, ctx->w, ctx->pf_w, st))) return rc;
  if (rq_batch_weight_bytes(ctx->cfg, FUSED_NWG)) {
    vui_weights wt;
    if ((rc = rq_batch_tile_weights(ctx->cfg, ctx->w, ctx->rq_tw, &wt, st))) return rc;
    HIP_TRY(hipMemcpyAsync(ctx->wdev_t, &wt, sizeof(vui_weights), hipMemcpyHostToDevice, st));
    HIP_TRY(hipStreamSynchronize(st));  // wt is a local
  }
  HIP_TRY(hipStreamSynchronize(st));
  ctx->fused_ok = 0;
  ctx->fused_why[0] = 0;
  ctx->ns = FUSED_NS;
  ctx->lds_bytes = frame_lds_bytes(ctx->cfg);
  int n_cu = 0;
  ctx->nwg = FUSED_NWG;
  if (frame_supported(ctx->cfg, ctx->nwg, ctx->ns, true, ctx->fused_why, sizeof(ctx->fused_why))) {
    const int cap = frame_max_resident(ctx->lds_bytes, &n_cu);
    if (cap < 0) return cap;
    if (cap >= ctx->nwg) ctx->fused_ok = 1;
    else snprintf(ctx->fused_why, sizeof(ctx->fused_why), "only %d workgroups can be resident (%d CUs), %d needed", cap, n_cu, ctx->nwg);
  }
  // a depth head whose keys/values do not fit in LDS still leaves the backbone step to the one-launch kernel
  ctx->fused_bb_ok = ctx->fused_ok;
  ctx->lds_bb = ctx->lds_bytes;
  if (!ctx->fused_ok && frame_supported(ctx->cfg, ctx->nwg, ctx->ns, false, nullptr, 0)) {
    ctx->lds_bb = frame_lds_bytes_backbone(ctx->cfg);
    const int cap = frame_max_resident(ctx->lds_bb, &n_cu);
    if (cap < 0) return cap;
    if (cap >= ctx->nwg) ctx->fused_bb_ok = 1;
  }
  ctx->bb_ok = 0;
  ctx->bb_why[0] = 0;
  if (bb_batch_supported(ctx->cfg, ctx->nwg, ctx->bb_why, sizeof(ctx->bb_why))) {
    ctx->bb_w8_bytes = bb_batch_weight_bytes(ctx->cfg, ctx->nwg);
    if ((rc = bb_batch_tile_weights(ctx->cfg, ctx->w, ctx->bb_w8_bytes ? ctx->bb_w8 : nullptr, ctx->bb_head, st))) return rc;
    HIP_TRY(hipStreamSynchronize(st));
    const int cap = bb_batch_max_resident(ctx->cfg);
    if (cap < 0) return cap;
    if (cap >= ctx->nwg) ctx->bb_ok = 1;
    else snprintf(ctx->bb_why, sizeof(ctx->bb_why), "only %d workgroups can be resident, %d needed", cap, ctx->nwg);
  }
  ctx->rqb_ok = 0;
  ctx->rqb_why[0] = 0;
  if (rq_batch_supported(ctx->cfg, ctx->nwg, ctx->rqb_why, sizeof(ctx->rqb_why))) {
    const int cap = rq_batch_max_resident(rq_batch_lds_bytes(ctx->cfg));
    if (cap < 0) return cap;
    if (cap >= ctx->nwg) ctx->rqb_ok = 1;
    else snprintf(ctx->rqb_why, sizeof(ctx->rqb_why), "only %d workgroups can be resident, %d needed", cap, ctx->nwg);
  }
  return VUI_OK;
}

// ---- a share of the GPU for the one-launch kernel ----
int vui_cu_stream_create(int first_cu, int n_cus, vui_stream_t* out) {
  if (!out) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  int dev = 0, cus = 0;
  HIP_TRY(hipGetDevice(&dev));
  HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  if (first_cu < 0 || n_cus < 1 || first_cu + n_cus > cus || cus > 1024) { vui_set_error("compute units [%d, %d) outside [0, %d)", first_cu, first_cu + n_cus, cus); return VUI_EINVAL; }
  uint32_t mask[32];
  memset(mask, 0, sizeof(mask));
  for (int b = first_cu; b < first_cu + n_cus; ++b) mask[b >> 5] |= 1u << (b & 31);
  hipStream_t st = nullptr;
  HIP_TRY(hipExtStreamCreateWithCUMask(&st, (uint32_t)((cus + 31) / 32), mask));
  *out = (vui_stream_t)st;
  return VUI_OK;
}

int vui_ctx_workgroups(vui_ctx* ctx, int nwg) {
  if (!ctx) { vui_set_error("NULL context"); return VUI_EINVAL; }
  const vui_config& c = ctx->cfg;
  if (!ctx->fused_ok) { vui_set_error("the one-launch kernel is not available: %s", ctx->fused_why); return VUI_EINVAL; }
  // A persistent kernel on a stream bound to part of the GPU needs every workgroup resident on the compute units of its
  // range.  The dispatcher deals workgroups evenly over the shader engines of every XCD, so the range must leave every
  // engine the same number of compute units: multiples of 32 (8 XCDs x 4 engines).  On 144 and 152 units (18 and 19 per
  // XCD) the launch ended in its bounded wait, while the same 152 workgroups on the whole GPU ran: one engine was asked
  // for more resident workgroups than it had units.  160 is the fewest the widest matrix of Vui Nano allows.
  if (nwg < 160 || nwg > FUSED_NWG || nwg % 32) { vui_set_error("workgroups %d: 160, 192, 224 or %d", nwg, FUSED_NWG); return VUI_EINVAL; }
  int ns = nwg / (c.n_heads > 0 ? c.n_heads : 1);
  if (ns > FUSED_NS) ns = FUSED_NS;
  char why[96] = "";
  if (ns < 1 || !frame_supported(c, nwg, ns, true, why, sizeof(why))) { vui_set_error("the one-launch kernel does not run on %d workgroups: %s", nwg, why[0] ? why : "too few for the heads"); return VUI_EINVAL; }
  ctx->nwg = nwg;
  ctx->ns = ns;
  if (nwg != FUSED_NWG) { ctx->rqb_ok = 0; ctx->bb_ok = 0; snprintf(ctx->rqb_why, sizeof(ctx->rqb_why), "the context was limited to %d workgroups", nwg); snprintf(ctx->bb_why, sizeof(ctx->bb_why), "the context was limited to %d workgroups", nwg); }
  return VUI_OK;
}

int vui_ctx_fused(vui_ctx* ctx, int enable) {
  if (!ctx) { vui_set_error("NULL context"); return VUI_EINVAL; }
  if (enable >= 0) ctx->fused_on = enable ? 1 : 0;
  if (!ctx->fused_ok && ctx->fused_why[0]) vui_set_error("fused frame kernel unavailable: %s", ctx->fused_why);
  return (ctx->fused_ok && ctx->fused_on) ? 1 : 0;
}

int vui_ctx_rq_batch(vui_ctx* ctx) {
  if (!ctx) { vui_set_error("NULL context"); return VUI_EINVAL; }
  if (!ctx->rqb_ok && ctx->rqb_why[0]) vui_set_error("batched depth-head kernel unavailable: %s", ctx->rqb_why);
  return (ctx->rqb_ok && ctx->fused_on) ? 1 : 0;
}

int vui_debug_phase_clock(vui_ctx* ctx, uint64_t* buf, int cap, int workgroup) {
  if (!ctx) { vui_set_error("NULL context"); return VUI_EINVAL; }
  ctx->prof = buf; ctx->prof_cap = buf ? cap : 0; ctx->prof_wg = workgroup;
  return VUI_OK;
}

int vui_ctx_bb_batch(vui_ctx* ctx) {
  if (!ctx) { vui_set_error("NULL context"); return VUI_EINVAL; }
  if (!ctx->bb_ok && ctx->bb_why[0]) vui_set_error("batched backbone kernel unavailable: %s", ctx->bb_why);
  return (ctx->bb_ok && ctx->fused_on) ? 1 : 0;
}

int vui_debug_set_epoch(vui_ctx* ctx, uint32_t value) {
  if (!ctx) { vui_set_error("NULL context"); return VUI_EINVAL; }
  HIP_TRY(hipDeviceSynchronize());
  HIP_TRY(hipMemcpy(ctx->ctl, &value, sizeof(value), hipMemcpyHostToDevice));
  return VUI_OK;
}

int vui_ctx_status(vui_ctx* ctx) {
  if (!ctx) { vui_set_error("NULL context"); return VUI_EINVAL; }
  uint32_t h[4] = {0, 0, 0, 0};
  HIP_TRY(hipMemcpy(h, ctx->ctl, sizeof(h), hipMemcpyDeviceToHost));
  if (h[2] == 2) { vui_set_error("persistent kernel: the launch count wrapped (epoch %u); call vui_ctx_init again", h[0]); return VUI_EHIP; }
  if (h[2]) { vui_set_error("persistent kernel: an exchange wait timed out (epoch %u); was another kernel running on the device? call vui_ctx_init again", h[0]); return VUI_EHIP; }
  return VUI_OK;
}

static void fused_base(vui_ctx* ctx, FrameArgs& a) {
  const vui_config& c = ctx->cfg;
  memset(&a, 0, sizeof(a));
  a.d = c.d_model; a.L = c.n_layers; a.H = c.n_heads; a.KV = c.n_kv_heads; a.hd = c.head_dim; a.F = c.ffn;
  a.Q = c.n_quantizers; a.CS = c.codebook_size; a.R = c.rq_dim; a.rqL = c.rq_layers; a.rqH = c.rq_heads; a.rqF = c.rq_ffn;
  a.rope_dim = c.rope_dim; a.S = c.max_seqlen; a.window = c.window; a.eps = c.norm_eps; a.rq_eps = c.rq_norm_eps;
  a.w = ctx->wdev; a.n_slots = c.n_slots;
  a.global_layers = c.global_layers; a.global_rope_dim = c.global_rope_dim;
  a.ll = ctx->ll; a.epoch = ctx->ctl; a.arrive = ctx->ctl + 1; a.err = ctx->ctl + 2;
  a.prof = ctx->prof; a.prof_cap = ctx->prof_cap; a.prof_wg = ctx->prof_wg;
  a.ns = ctx->ns; a.lds_kv_off = (int)(ctx->lds_bytes - frame_rq_lds_cache_bytes(c));
  a.rq_kg = frame_rq_keys_global(c); a.rq_kscratch = (uint16_t*)ctx->rq_ks; a.w_int8 = c.int8_backbone;
}
static bool use_fused(vui_ctx* ctx, int B) { return ctx->fused_ok && ctx->fused_on && B == 1; }

static int check_batch(vui_ctx* ctx, int B, int n_splits) {
  if (!ctx) { vui_set_error("NULL context"); return VUI_EINVAL; }
  if (B < 1 || B > ctx->max_batch) { vui_set_error("B=%d outside [1, max_batch=%d]", B, ctx->max_batch); return VUI_EINVAL; }
  if (n_splits < 1 || n_splits > MAX_SPLITS) { vui_set_error("n_splits=%d outside [1,%d]", n_splits, MAX_SPLITS); return VUI_EINVAL; }
  return VUI_OK;
}

int64_t vui_prefill_scratch_bytes(const vui_config* c, int T, int L) {
  if (!c || T < 1 || L < T) { vui_set_error("vui_prefill_scratch_bytes: bad arguments"); return VUI_EINVAL; }
  char why[96];
  if (!prefill_supported(*c, why, sizeof(why))) { vui_set_error("prefill pass unavailable: %s", why); return VUI_EINVAL; }
  return (int64_t)prefill_scratch_bytes(*c, T, L);
}

int vui_prefill(vui_ctx* ctx, const void* emb_in, int T, int slot, int pos0, int32_t* seq_lens, void* k_cache, void* v_cache,
                void* hidden_out, void* scratch, int64_t scratch_bytes, vui_stream_t stream) {
  if (!ctx) { vui_set_error("NULL context"); return VUI_EINVAL; }
  if (!emb_in || !seq_lens || !k_cache || !v_cache || !hidden_out || !scratch) { vui_set_error("vui_prefill: NULL argument"); return VUI_EINVAL; }
  if (((uintptr_t)scratch & 255) || scratch_bytes < 0) { vui_set_error("vui_prefill: scratch must be 256-byte aligned"); return VUI_EINVAL; }
  const void* tiled = prefill_weight_bytes(ctx->cfg) ? ctx->pf_w : ((ctx->cfg.int8_backbone && ctx->bb_w8_bytes) ? ctx->bb_w8 : nullptr);
  return launch_prefill(ctx->cfg, ctx->w, tiled, emb_in, T, slot, pos0, seq_lens, k_cache,
                        v_cache, hidden_out, scratch, (size_t)scratch_bytes, (hipStream_t)stream);
}

int vui_backbone_step(vui_ctx* ctx, const int64_t* codes_in, const void* emb_in, const int32_t* slot_idx,
                      int32_t* seq_lens, const int32_t* seq_inc, int B, void* k_cache, void* v_cache, void* hidden_out,
                      void* cb0_out, void* eos_out, int n_splits, vui_stream_t stream) {
  int rc = check_batch(ctx, B, n_splits);
  if (rc) return rc;
  if ((codes_in == nullptr) == (emb_in == nullptr)) { vui_set_error("exactly one of codes_in / emb_in must be given"); return VUI_EINVAL; }
  if (!seq_lens || !k_cache || !v_cache) { vui_set_error("seq_lens and the KV caches are required"); return VUI_EINVAL; }
  const vui_config& c = ctx->cfg;
  hipStream_t st = (hipStream_t)stream;
  if (ctx->fused_bb_ok && ctx->fused_on && B == 1) {
    FrameArgs a;
    fused_base(ctx, a);
    a.mode = FR_BACKBONE;
    a.codes_in = codes_in; a.emb_in = (const uint16_t*)emb_in; a.slot_idx = slot_idx; a.seq_lens = seq_lens; a.seq_inc = seq_inc;
    a.kc = (uint16_t*)k_cache; a.vc = (uint16_t*)v_cache;
    a.hidden_out = (uint16_t*)(hidden_out ? hidden_out : ctx->hidden);
    a.cb0_out = (uint16_t*)(cb0_out ? cb0_out : ctx->cb0);
    a.eos_out = (uint16_t*)(eos_out ? eos_out : ctx->eos);
    if (!ctx->fused_ok) a.lds_kv_off = (int)ctx->lds_bb;  // no depth-head cache in this launch
    return launch_frame(a, ctx->nwg, ctx->fused_ok ? ctx->lds_bytes : ctx->lds_bb, st);
  }
  if (ctx->bb_ok && ctx->fused_on && B > 1)
    return launch_bb_batch(c, ctx->wdev, ctx->bb_w8_bytes ? ctx->bb_w8 : ctx->pf_w, ctx->bb_head, codes_in, emb_in, slot_idx, seq_lens, seq_inc, B,
                           k_cache, v_cache, hidden_out ? hidden_out : ctx->hidden, cb0_out ? cb0_out : ctx->cb0,
                           eos_out ? eos_out : ctx->eos, ctx->ll, ctx->ctl, ctx->nwg, st);
  const int d = c.d_model, H = c.n_heads, KV = c.n_kv_heads, hd = c.head_dim;
  if (codes_in) rc = launch_embed(c.dtype, codes_in, ctx->w.audio_emb, ctx->x, B, c.n_quantizers, c.codebook_size, d, st);
  else rc = launch_copy_rows(c.dtype, emb_in, ctx->x, (int64_t)B * d, st);
  if (rc) return rc;
  const size_t slab = (size_t)c.n_slots * c.max_seqlen * KV * hd * ctx->esz;
  for (int l = 0; l < c.n_layers; ++l) {
    const vui_layer_weights& L = ctx->w.layers[l];
    void* kc = (char*)k_cache + slab * l;
    void* vc = (char*)v_cache + slab * l;
    GemvArgs g;
    memset(&g, 0, sizeof(g));
    g.dtype = c.dtype; g.w_int8 = c.int8_backbone;
    g.x = ctx->x; g.norm_w = L.attn_norm; g.eps = c.norm_eps;
    g.W = L.wqkv; g.sc = L.s_qkv; g.y = ctx->q; g.ldy = H * hd;
    g.B = B; g.N = (H + 2 * KV) * hd; g.K = d; g.epi = EPI_QKV;
    g.rope = layer_rope(c, ctx->w, l, &g.rope_dim); g.hd = hd; g.nq = H * hd; g.nkv = KV * hd;
    g.kc = kc; g.vc = vc; g.seq_lens = seq_lens; g.slot_idx = slot_idx; g.S = c.max_seqlen;
    if ((rc = launch_gemv(g, st))) return rc;

    AttnArgs a;
    memset(&a, 0, sizeof(a));
    a.dtype = c.dtype; a.q = ctx->q; a.kc = kc; a.vc = vc; a.seq_lens = seq_lens; a.slot_idx = slot_idx;
    a.out = ctx->att; a.B = B; a.H = H; a.KV = KV; a.hd = hd; a.S = c.max_seqlen; a.window = layer_window(c, l);
    a.n_splits = n_splits; a.part = ctx->part; a.counter = ctx->counter;
    if ((rc = launch_decode_attn(a, st))) return rc;

    memset(&g, 0, sizeof(g));
    g.dtype = c.dtype; g.w_int8 = c.int8_backbone;
    g.x = ctx->att; g.W = L.wo; g.sc = L.s_o; g.y = ctx->x; g.resid = ctx->x; g.ldy = d;
    g.B = B; g.N = d; g.K = d; g.epi = EPI_RESID;
    if ((rc = launch_gemv(g, st))) return rc;

    memset(&g, 0, sizeof(g));
    g.dtype = c.dtype; g.w_int8 = c.int8_backbone;
    g.x = ctx->x; g.norm_w = L.mlp_norm; g.eps = c.norm_eps;
    g.W = L.w1; g.W2 = L.w3; g.sc = L.s_1; g.sc2 = L.s_3; g.y = ctx->h; g.ldy = c.ffn;
    g.B = B; g.N = c.ffn; g.K = d; g.epi = EPI_SWIGLU;
    if ((rc = launch_gemv(g, st))) return rc;

    memset(&g, 0, sizeof(g));
    g.dtype = c.dtype; g.w_int8 = c.int8_backbone;
    g.x = ctx->h; g.W = L.w2; g.sc = L.s_2; g.y = ctx->x; g.resid = ctx->x; g.ldy = d;
    g.B = B; g.N = d; g.K = c.ffn; g.epi = EPI_RESID;
    if ((rc = launch_gemv(g, st))) return rc;
  }
  // final norm + codec_head (+ eos head, hidden output and position update in the extra block)
  GemvArgs g;
  memset(&g, 0, sizeof(g));
  g.dtype = c.dtype;
  g.x = ctx->x; g.norm_w = ctx->w.final_norm; g.eps = c.norm_eps;
  g.W = ctx->w.codec_head; g.y = cb0_out ? cb0_out : ctx->cb0; g.ldy = c.codebook_size;
  g.B = B; g.N = c.codebook_size; g.K = d; g.epi = EPI_STORE;
  g.Wx = ctx->w.eos_w; g.bx = ctx->w.eos_b; g.yx = eos_out ? eos_out : ctx->eos;
  g.hid_out = hidden_out ? hidden_out : ctx->hidden;
  g.upd_seq_lens = seq_lens; g.upd_seq_inc = seq_inc; g.slot_idx = slot_idx; g.n_slots = c.n_slots;
  return launch_gemv(g, st);
}

static SampleArgs sample_base(const vui_sample_params* sp) {
  SampleArgs s;
  memset(&s, 0, sizeof(s));
  s.temperature = sp->temperature; s.top_k = sp->top_k; s.seed = sp->seed; s.frame_ctr = sp->frame_ctr;
  s.state_rows = sp->state_rows; s.top_p = sp->top_p; s.dev = sp->dev;
  return s;
}

int vui_sample_cb0(vui_ctx* ctx, const void* logits, float* rep_counts, int32_t* rep_hist, int32_t* rep_pos,
                   float penalty, int window, const vui_sample_params* sp, int64_t* code0_out, int B,
                   vui_stream_t stream) {
  int rc = check_batch(ctx, B, 1);
  if (rc) return rc;
  if (!logits || !sp || !code0_out) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  if (window > 0 && rep_counts && penalty > 1.0f && (!rep_hist || !rep_pos)) { vui_set_error("a repetition window needs rep_hist and rep_pos"); return VUI_EINVAL; }
  SampleArgs s = sample_base(sp);
  s.dtype = ctx->cfg.dtype; s.logits = logits; s.rep_counts = rep_counts; s.rep_hist = rep_hist; s.rep_pos = rep_pos;
  s.penalty = penalty; s.window = window; s.codebook = 0; s.exact_k = sp->keep_ties ? 0 : 1; s.CS = ctx->cfg.codebook_size; s.B = B;
  s.out = code0_out; s.out_stride = 1; s.out_col = 0;
  return launch_sample(s, (hipStream_t)stream);
}

static int rq_layers_step(vui_ctx* ctx, int B, int pos, bool kv_only_last, hipStream_t st) {
  const vui_config& c = ctx->cfg;
  const int R = c.rq_dim, Q = c.n_quantizers;
  int rc;
  for (int l = 0; l < c.rq_layers; ++l) {
    const vui_rq_layer_weights& L = ctx->w.rq_layers[l];
    const size_t lay = (size_t)ctx->max_batch * Q * R * ctx->esz;
    GemvArgs g;
    memset(&g, 0, sizeof(g));
    g.dtype = c.dtype; g.x = ctx->rx; g.norm_w = L.attn_norm; g.eps = c.rq_norm_eps;
    g.W = L.wqkv; g.y = ctx->rq_q; g.ldy = R; g.B = B; g.N = 3 * R; g.K = R; g.epi = EPI_RQ_QKV;
    g.nq = R; g.kc = (char*)ctx->rq_kc + lay * l; g.vc = (char*)ctx->rq_vc + lay * l; g.S = Q; g.rq_pos = pos;
    if ((rc = launch_gemv(g, st))) return rc;
    if (kv_only_last && l == c.rq_layers - 1) break;  // position 0 only feeds later keys/values

    RqAttnArgs a;
    memset(&a, 0, sizeof(a));
    a.dtype = c.dtype; a.q = ctx->rq_q; a.kc = g.kc; a.vc = g.vc; a.out = ctx->rq_att;
    a.B = B; a.heads = c.rq_heads; a.hd = R / c.rq_heads; a.Q = Q; a.pos = pos;
    if ((rc = launch_rq_attn(a, st))) return rc;

    memset(&g, 0, sizeof(g));
    g.dtype = c.dtype; g.x = ctx->rq_att; g.W = L.wo; g.y = ctx->rx; g.resid = ctx->rx; g.ldy = R;
    g.B = B; g.N = R; g.K = R; g.epi = EPI_RESID;
    if ((rc = launch_gemv(g, st))) return rc;

    memset(&g, 0, sizeof(g));
    g.dtype = c.dtype; g.x = ctx->rx; g.norm_w = L.mlp_norm; g.eps = c.rq_norm_eps;
    g.W = L.w1; g.W2 = L.w3; g.y = ctx->rq_h; g.ldy = c.rq_ffn; g.B = B; g.N = c.rq_ffn; g.K = R; g.epi = EPI_SWIGLU;
    if ((rc = launch_gemv(g, st))) return rc;

    memset(&g, 0, sizeof(g));
    g.dtype = c.dtype; g.x = ctx->rq_h; g.W = L.w2; g.y = ctx->rx; g.resid = ctx->rx; g.ldy = R;
    g.B = B; g.N = R; g.K = c.rq_ffn; g.epi = EPI_RESID;
    if ((rc = launch_gemv(g, st))) return rc;
  }
  return VUI_OK;
}

int vui_rq_generate(vui_ctx* ctx, const void* hidden, const int64_t* code0, const float* logit_bias, int n_q,
                    const vui_sample_params* sp, int64_t* codes_out, int codes_stride, int zero_pad, int B,
                    vui_stream_t stream) {
  int rc = check_batch(ctx, B, 1);
  if (rc) return rc;
  const vui_config& c = ctx->cfg;
  if (c.rq_layers < 1) { vui_set_error("context has no depth head"); return VUI_EINVAL; }
  if (!hidden || !code0 || !sp || !codes_out) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  if (n_q < 2 || n_q > c.n_quantizers || codes_stride < n_q) { vui_set_error("n_q=%d outside [2,%d] or stride %d too small", n_q, c.n_quantizers, codes_stride); return VUI_EINVAL; }
  if (sp->top_p > 0.f) { vui_set_error("the depth head draws with temperature and top-k only (model.py:955-962): top_p must be 0"); return VUI_EINVAL; }
  hipStream_t st = (hipStream_t)stream;
  if (use_fused(ctx, B)) {
    FrameArgs a;
    fused_base(ctx, a);
    a.mode = FR_RQ;
    a.rq_hidden = (const uint16_t*)hidden; a.rq_code0 = code0; a.logit_bias = logit_bias; a.n_q = n_q;
    a.temp1 = sp->temperature; a.topk1 = sp->top_k; a.seed1 = sp->seed; a.frame_ctr1 = sp->frame_ctr; a.sdev1 = sp->dev;
    a.codes_out = codes_out; a.codes_stride = codes_stride; a.zero_pad = zero_pad;
    return launch_frame(a, ctx->nwg, ctx->lds_bytes, st);
  }
  if (ctx->rqb_ok && ctx->fused_on && B > 1)
    return launch_rq_batch(c, ctx->wdev_t, hidden, code0, logit_bias, n_q, sp->temperature, sp->top_k, sp->seed, sp->dev, sp->frame_ctr,
                           codes_out, codes_stride, zero_pad, B, ctx->ll, ctx->ctl, ctx->nwg, st);
  const int R = c.rq_dim, CS = c.codebook_size;
  const char* pos_emb = (const char*)ctx->w.rq_pos_emb;
  const size_t rowb = (size_t)R * ctx->esz;

  // position 0: projected backbone hidden + pos_emb[0]   (model.py:921)
  if (ctx->w.rq_backbone_proj) {
    GemvArgs g;
    memset(&g, 0, sizeof(g));
    g.dtype = c.dtype; g.x = hidden; g.W = ctx->w.rq_backbone_proj; g.y = ctx->rx; g.ldy = R; g.vec = pos_emb;
    g.B = B; g.N = R; g.K = c.d_model; g.epi = EPI_ADDVEC;
    if ((rc = launch_gemv(g, st))) return rc;
  } else {
    if ((rc = launch_add_rows(c.dtype, hidden, pos_emb, ctx->rx, B, R, st))) return rc;
  }
  if ((rc = rq_layers_step(ctx, B, 0, true, st))) return rc;
  // position 1: code-0 embedding + pos_emb[1]   (model.py:922-925); also codes_out[:, 0] = code0
  if ((rc = launch_rq_token(c.dtype, code0, 0, ctx->w.rq_code_emb, pos_emb + rowb, ctx->rx, B, R, codes_out,
                            codes_stride, CS, st)))
    return rc;
  for (int i = 0; i < n_q - 1; ++i) {
    if ((rc = rq_layers_step(ctx, B, i + 1, false, st))) return rc;
    GemvArgs g;
    memset(&g, 0, sizeof(g));
    g.dtype = c.dtype; g.x = ctx->rx; g.norm_w = ctx->w.rq_norm; g.eps = c.rq_norm_eps;
    g.W = (const char*)ctx->w.rq_head_w + (size_t)i * CS * rowb; g.y = ctx->rq_logits; g.ldy = CS;
    g.B = B; g.N = CS; g.K = R; g.epi = EPI_STORE;
    if ((rc = launch_gemv(g, st))) return rc;
    SampleArgs s = sample_base(sp);
    s.dtype = c.dtype; s.logits = ctx->rq_logits; s.bias = logit_bias ? logit_bias + (size_t)i * CS : nullptr;
    s.codebook = i + 1; s.CS = CS; s.B = B; s.out = codes_out; s.out_stride = codes_stride; s.out_col = i + 1;
    const bool last = (i == n_q - 2);
    if (!last) {
      s.tok_emb = ctx->w.rq_code_emb; s.tok_emb_off = (int64_t)(i + 1) * CS; s.tok_pos = pos_emb + rowb * (i + 2);
      s.tok_out = ctx->rx; s.R = R;
    } else if (zero_pad) {
      s.pad_from = n_q; s.pad_to = codes_stride;
    }
    if ((rc = launch_sample(s, st))) return rc;
  }
  return VUI_OK;
}

int vui_frame_step(vui_ctx* ctx, int64_t* codes_io, const int32_t* slot_idx, int32_t* seq_lens, const int32_t* seq_inc,
                   int B, void* k_cache, void* v_cache, float* rep_counts, int32_t* rep_hist, int32_t* rep_pos,
                   float penalty, int window, const vui_sample_params* sp_cb0, const vui_sample_params* sp_rq,
                   const float* logit_bias, int n_q, void* hidden_out, void* cb0_out, float* eos_prob_out,
                   int64_t* frames_out, int max_frames, int32_t* frame_ctr, int n_splits, const vui_eos_stop* stop,
                   vui_stream_t stream) {
  int rc = check_batch(ctx, B, n_splits);
  if (rc) return rc;
  if (!codes_io || !sp_cb0 || !sp_rq || !frame_ctr) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  if (stop && (B != 1 || !stop->state)) { vui_set_error("the device-side end-of-turn test takes one row and a state pointer"); return VUI_EINVAL; }
  const vui_config& c = ctx->cfg;
  hipStream_t st = (hipStream_t)stream;
  void* hid = hidden_out ? hidden_out : ctx->hidden;
  void* cb0 = cb0_out ? cb0_out : ctx->cb0;
  if (window > 0 && rep_counts && penalty > 1.0f && (!rep_hist || !rep_pos)) { vui_set_error("a repetition window needs rep_hist and rep_pos"); return VUI_EINVAL; }
  if (n_q < 2 || n_q > c.n_quantizers) { vui_set_error("n_q=%d outside [2,%d]", n_q, c.n_quantizers); return VUI_EINVAL; }
  if (sp_cb0->top_p > 0.f || sp_rq->top_p > 0.f) { vui_set_error("vui_frame_step is Engine's step, whose samplers have no nucleus cut: top_p must be 0 (vui_sample_cb0 takes it)"); return VUI_EINVAL; }
  if (use_fused(ctx, B)) {
    if (!seq_lens || !k_cache || !v_cache) { vui_set_error("seq_lens and the KV caches are required"); return VUI_EINVAL; }
    FrameArgs a;
    fused_base(ctx, a);
    a.mode = FR_BACKBONE | FR_CB0 | FR_RQ | FR_FINISH;
    a.codes_in = codes_io; a.slot_idx = slot_idx; a.seq_lens = seq_lens; a.seq_inc = seq_inc;
    a.kc = (uint16_t*)k_cache; a.vc = (uint16_t*)v_cache;
    a.hidden_out = (uint16_t*)hid; a.cb0_out = (uint16_t*)cb0; a.eos_out = (uint16_t*)ctx->eos;
    a.rep_counts = rep_counts; a.rep_hist = rep_hist; a.rep_pos = rep_pos; a.penalty = penalty; a.rep_window = window;
    a.temp0 = sp_cb0->temperature; a.topk0 = sp_cb0->top_k; a.seed0 = sp_cb0->seed; a.frame_ctr0 = sp_cb0->frame_ctr;
    a.temp1 = sp_rq->temperature; a.topk1 = sp_rq->top_k; a.seed1 = sp_rq->seed; a.frame_ctr1 = sp_rq->frame_ctr;
    a.sdev0 = sp_cb0->dev; a.sdev1 = sp_rq->dev;
    a.code0_out = ctx->code0; a.logit_bias = logit_bias; a.n_q = n_q;
    a.codes_out = codes_io; a.codes_stride = c.n_quantizers; a.zero_pad = 1;
    a.frames_out = frames_out; a.eos_prob_out = eos_prob_out; a.max_frames = max_frames; a.frame_ctr = frame_ctr;
    a.exact0 = sp_cb0->keep_ties ? 0 : 1;
    if (stop) { a.stop_state = stop->state; a.stop_thr = stop->threshold; a.stop_min = stop->min_frames; }
    return launch_frame(a, ctx->nwg, ctx->lds_bytes, st);
  }
  if ((rc = vui_backbone_step(ctx, codes_io, nullptr, slot_idx, seq_lens, seq_inc, B, k_cache, v_cache, hid, cb0,
                              ctx->eos, n_splits, stream)))
    return rc;
  if (window > 0 && rep_counts && penalty > 1.0f && (!rep_hist || !rep_pos)) { vui_set_error("a repetition window needs rep_hist and rep_pos"); return VUI_EINVAL; }
  SampleArgs s = sample_base(sp_cb0);
  s.dtype = c.dtype; s.logits = cb0; s.rep_counts = rep_counts; s.rep_hist = rep_hist; s.rep_pos = rep_pos;
  s.penalty = penalty; s.window = window; s.codebook = 0; s.exact_k = sp_cb0->keep_ties ? 0 : 1; s.CS = c.codebook_size; s.B = B;
  s.out = ctx->code0; s.out_stride = 1; s.out_col = 0;
  s.eos_logit = ctx->eos; s.eos_prob = ctx->eos_prob;
  if ((rc = launch_sample(s, st))) return rc;
  if ((rc = vui_rq_generate(ctx, hid, ctx->code0, logit_bias, n_q, sp_rq, codes_io, c.n_quantizers, 1, B, stream)))
    return rc;
  return launch_frame_finish(codes_io, frames_out, B * c.n_quantizers, max_frames, frame_ctr, ctx->eos_prob,
                             eos_prob_out, B, stop ? stop->state : nullptr, stop ? stop->threshold : 0.f,
                             stop ? stop->min_frames : 0, st);
}

// ---- HIP graphs ----
struct vui_graph {
  hipGraph_t graph;
  hipGraphExec_t exec;
};

int vui_graph_begin(vui_stream_t stream) {
  HIP_TRY(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
  return VUI_OK;
}

int vui_graph_end(vui_stream_t stream, vui_graph** out) {
  hipGraph_t g = nullptr;
  HIP_TRY(hipStreamEndCapture((hipStream_t)stream, &g));
  if (!out || !g) { if (g) (void)hipGraphDestroy(g); vui_set_error("capture produced no graph"); return VUI_EINVAL; }
  hipGraphExec_t e = nullptr;
  hipError_t err = hipGraphInstantiate(&e, g, nullptr, nullptr, 0);
  if (err != hipSuccess) { (void)hipGraphDestroy(g); vui_set_error("hipGraphInstantiate failed: %s", hipGetErrorString(err)); return VUI_EHIP; }
  vui_graph* vg = new (std::nothrow) vui_graph();
  if (!vg) { (void)hipGraphExecDestroy(e); (void)hipGraphDestroy(g); vui_set_error("out of host memory"); return VUI_ENOMEM; }
  vg->graph = g; vg->exec = e;
  *out = vg;
  return VUI_OK;
}

int vui_graph_launch(vui_graph* g, vui_stream_t stream) {
  if (!g) { vui_set_error("NULL graph"); return VUI_EINVAL; }
  HIP_TRY(hipGraphLaunch(g->exec, (hipStream_t)stream));
  return VUI_OK;
}

void vui_graph_destroy(vui_graph* g) {
  if (!g) return;
  (void)hipGraphExecDestroy(g->exec);
  (void)hipGraphDestroy(g->graph);
  delete g;
}

// ---- single kernels ----
int vui_rmsnorm_gemv(int dtype, const void* x, const void* norm_w, float eps, const void* W, const void* scales,
                     int w_int8, void* y, int B, int N, int K, vui_stream_t stream) {
  if (!x || !W || !y || (w_int8 && !scales)) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  if (B > VUI_MAX_BATCH) { vui_set_error("B=%d > %d", B, VUI_MAX_BATCH); return VUI_EINVAL; }
  GemvArgs g;
  memset(&g, 0, sizeof(g));
  g.dtype = dtype; g.w_int8 = w_int8; g.x = x; g.norm_w = norm_w; g.eps = eps; g.W = W; g.sc = scales;
  g.y = y; g.ldy = N; g.B = B; g.N = N; g.K = K; g.epi = EPI_STORE;
  return launch_gemv(g, (hipStream_t)stream);
}

int vui_rope(int dtype, void* x, const float* rope_table, const int32_t* pos, int B, int n_heads, int head_dim,
             int rope_dim, vui_stream_t stream) {
  if (!x || !rope_table || !pos) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  return launch_rope(dtype, x, rope_table, pos, B, n_heads, head_dim, rope_dim, (hipStream_t)stream);
}

int64_t vui_attn_scratch_bytes(int B, int H, int hd, int n_splits) {
  return (int64_t)B * H * 256 + (int64_t)B * H * n_splits * (hd + 2) * 4;
}

int vui_decode_attn(int dtype, const void* q, const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                    const int32_t* seq_lens, const int32_t* slot_idx, void* out, int B, int H, int KV, int hd, int S,
                    int window, int n_splits, void* scratch, vui_stream_t stream) {
  if (!q || !k_cache || !v_cache || !seq_lens || !out || !scratch) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  int rc;
  if (k_new && v_new)
    if ((rc = launch_kv_append(dtype, k_new, v_new, k_cache, v_cache, seq_lens, slot_idx, B, KV, hd, S, (hipStream_t)stream)))
      return rc;
  AttnArgs a;
  memset(&a, 0, sizeof(a));
  a.dtype = dtype; a.q = q; a.kc = k_cache; a.vc = v_cache; a.seq_lens = seq_lens; a.slot_idx = slot_idx; a.out = out;
  a.B = B; a.H = H; a.KV = KV; a.hd = hd; a.S = S; a.window = window; a.n_splits = n_splits;
  a.counter = (uint32_t*)scratch;
  a.part = (float*)((char*)scratch + (size_t)B * H * 256);
  return launch_decode_attn(a, (hipStream_t)stream);
}

int vui_decode_attn_noalloc(int dtype, const void* q, const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                            const int32_t* seq_lens, const int32_t* slot_idx, void* out, int B, int H, int KV, int hd, int S,
                            int window, int n_splits, vui_stream_t stream) {
  if (!q || !k_cache || !v_cache || !seq_lens || !out) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  if (B < 1 || H < 1 || n_splits < 1 || hd < 8) { vui_set_error("decode_attn_noalloc: bad shape B=%d H=%d hd=%d splits=%d", B, H, hd, n_splits); return VUI_EINVAL; }
  const int64_t bh = (int64_t)B * H, pieces = bh * n_splits * (hd + 2) * 4;
  if (bh > NOALLOC_MAX_ROWS_HEADS || pieces > (int64_t)NOALLOC_PIECE_BYTES) {
    vui_set_error("decode_attn_noalloc: B*H=%lld (limit %d) with %d splits needs %lld bytes of pieces (limit %d): beyond the "
                  "built-in scratch, use vui_decode_attn with a scratch buffer of the caller",
                  (long long)bh, NOALLOC_MAX_ROWS_HEADS, n_splits, (long long)pieces, NOALLOC_PIECE_BYTES);
    return VUI_EINVAL;
  }
  unsigned char* sp = nullptr;
  int rc = noalloc_scratch(&sp);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  // the array keeps what the last call left: the arrival counters must start at zero (a fill kernel, so that the
  // call can be recorded into a graph)
  if (n_splits > 1 && (rc = launch_fill_u32((uint32_t*)sp, 0u, bh, st))) return rc;
  if (k_new && v_new)
    if ((rc = launch_kv_append(dtype, k_new, v_new, k_cache, v_cache, seq_lens, slot_idx, B, KV, hd, S, st))) return rc;
  AttnArgs a;
  memset(&a, 0, sizeof(a));
  a.dtype = dtype; a.q = q; a.kc = k_cache; a.vc = v_cache; a.seq_lens = seq_lens; a.slot_idx = slot_idx; a.out = out;
  a.B = B; a.H = H; a.KV = KV; a.hd = hd; a.S = S; a.window = window; a.n_splits = n_splits;
  a.counter = (uint32_t*)sp;
  a.part = (float*)(sp + (size_t)NOALLOC_MAX_ROWS_HEADS * 4);
  return launch_decode_attn(a, st);
}

int vui_sample_logits(const float* logits, const float* bias, int CS, const vui_sample_params* sp, int codebook,
                      int64_t* out, int B, vui_stream_t stream) {
  if (!logits || !sp || !out) { vui_set_error("NULL argument"); return VUI_EINVAL; }
  SampleArgs s = sample_base(sp);
  s.dtype = VUI_DTYPE_F32; s.logits = logits; s.bias = bias; s.codebook = codebook; s.CS = CS; s.B = B;
  s.out = out; s.out_stride = 1; s.out_col = 0;
  return launch_sample(s, (hipStream_t)stream);
}

}  // extern "C"
