/*
 * vui_codec.h - C ABI of the MI355X-native streaming vocoder frame step (codes of one codec frame ->
 * 1920 audio samples), the decoder half of the reference's codec.
 *
 * Same conventions as vui_amd.h: 0 on success, a negative VUI_E* code on failure with the message
 * in vui_last_error(); every pointer is a device pointer unless stated; all work is asynchronous
 * on the given HIP stream; the library allocates no device memory (the caller passes a workspace).
 * Arithmetic is fp32, the reference's codec regime (codec_dtype, src/vui/engine.py:302).
 *
 * Reference (paths relative to the reference checkout): QwenCodecDecoder._streaming_forward_body /
 * forward / _vocoder_chain (src/vui/qwen_codec.py:1191-1224) inside `decoder.streaming(1)`, as
 * driven one frame at a time by CodecCtx.decode_frame (qwen_codec.py:625-657).
 */
#ifndef VUI_CODEC_H
#define VUI_CODEC_H

#include "vui_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Architecture numbers of QwenCodecDecoder.__init__ (qwen_codec.py:1080-1125). */
typedef struct vui_codec_config {
  int32_t n_codebooks;   /* 16 */
  int32_t codebook_size; /* 2048 */
  int32_t codebook_dim;  /* 256 */
  int32_t vq_dim;        /* 512: width of the quantizer output projections */
  int32_t n_semantic;    /* 1: codebooks of the first residual group */
  int32_t latent_dim;    /* 1024 */
  int32_t d_model;       /* 512 */
  int32_t n_layers;      /* 8 */
  int32_t n_heads;       /* 16 */
  int32_t head_dim;      /* 64 */
  int32_t mlp_dim;       /* 1024 */
  int32_t max_seq;       /* 250: positions of the pre-transformer cache */
  float rope_theta;      /* 10000 */
  int32_t n_up;          /* 2 */
  int32_t up_ratios[4];  /* 2, 2 */
  int32_t decoder_dim;   /* 1536 */
  int32_t n_rates;       /* 4 */
  int32_t rates[8];      /* 8, 5, 4, 3 */
} vui_codec_config;

typedef struct vui_codec vui_codec;

/* Samples per frame: product of up_ratios and rates (1920).  Negative on an unsupported config. */
int32_t vui_codec_hop(const vui_codec_config* cfg);

/* Number of weight tensors vui_codec_init expects: the entries of QwenCodecDecoder.state_dict()
 * in its own order (quantizer.semantic.{input_proj.weight, output_proj.weight, codebooks.i.embed},
 * the same for quantizer.acoustic, pre_conv.conv.{weight,bias}, pre_transformer.*, upsample.*,
 * decoder.*; qwen_codec.py:1087-1125). */
int32_t vui_codec_n_tensors(const vui_codec_config* cfg);

/* Bytes of workspace: repacked weights (one copy, tap-major), activation rings, the
 * pre-transformer cache, tables and counters. */
int64_t vui_codec_workspace_bytes(const vui_codec_config* cfg);

/* Builds a decoder: repacks the fp32 tensors (reference layouts: Conv1d (out, in, k),
 * ConvTranspose1d (in, out, k), Linear (out, in)) into the workspace on `stream`; the caller's
 * tensors are not referenced afterwards.  The state starts cold.  Replaces
 * QwenCodecDecoder.from_pretrained + setup_streaming_graph (qwen_codec.py:1138-1189, 1278-1293). */
int vui_codec_init(const vui_codec_config* cfg, const void* const* tensors, int32_t n_tensors, void* workspace,
                   int64_t workspace_bytes, vui_stream_t stream, vui_codec** out);
void vui_codec_destroy(vui_codec* c);

/* Cold state: zero conv histories, position 0 - what entering `decoder.streaming(1)` afresh does
 * (CodecCtx._hard_reset, qwen_codec.py:609-623; _init_streaming_state :74-90, :122-138, :1011-1032). */
int vui_codec_reset(vui_codec* c, vui_stream_t stream);

/* One frame: codes (n_q) int64 of one codec frame -> audio_out (hop) fp32 in [-1, 1], advancing
 * every conv history and the pre-transformer cache by one frame.  n_q <= n_codebooks: the missing
 * codebooks are left out of the sum (SplitResidualVQ.decode, qwen_codec.py:263-270).  The call is
 * capturable into a HIP graph (position and histories advance on the device).  At most max_seq
 * frames between two resets; further frames raise the status flag and reuse the last position. */
int vui_codec_decode_frame(vui_codec* c, const int64_t* codes, int32_t n_q, float* audio_out, vui_stream_t stream);

/* The one-column steps of a frame (codebook rows ... first upsampling conv) run as one persistent kernel when
 * the device can keep 256 workgroups resident and the dimensions fit, otherwise as separate launches (same
 * sums in another order).  enable = 1/0 switches the persistent form on/off, -1 only queries; returns 1 when
 * it will be used, else 0.  No counterpart in the reference.  Do not run two persistent kernels of this library
 * (this one, the batch-1 frame kernel, the batched depth head) on different streams at the same time: each
 * needs all its workgroups resident. */
int vui_codec_persistent(vui_codec* c, int enable);

/* The persistent form on `nwg` workgroups instead of one per compute unit of the whole GPU, for a caller that runs
 * the vocoder on a stream bound to part of the GPU (vui_cu_stream_create of vui_amd.h) beside other work: the
 * kernel needs all its workgroups resident on the compute units its stream may use.  With fewer workgroups each
 * owns more rows of every matrix; below about 96 (at the reference's dims) the rows no longer fit the registers a
 * wave keeps them in and the call fails with VUI_EINVAL (vui_codec_persistent(c, 0) then runs the launches).
 * A vocoder limited this way reads its weights (each byte once per frame) with non-temporal loads, which leaves the
 * caches to the kernels it runs beside (measured: the decode step beside it 4 % faster; the vocoder alone would be
 * 4 % slower with them, so at the full width they are not used).
 * Steps captured earlier keep the width they were captured with.  No counterpart in the reference. */
int vui_codec_workgroups(vui_codec* c, int nwg);

/* Synchronous: frames decoded since the last reset (reads a device counter on `stream`), or a negative
 * code; VUI_EINVAL after a code outside [0, codebook_size) or a frame beyond max_seq was seen. */
int64_t vui_codec_status(vui_codec* c, vui_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
